"""Tensor-level entry points of the block top-k decode path.

Each function checks its tensors (dtype, device, contiguity, shape), then hands
raw device pointers and the current HIP stream to the C ABI
(include/kinetics_amd.h).  Nothing here computes: without the HIP library the
import of ``_lib`` fails.  The same functions are registered as
``torch.ops.kinetics.*`` custom ops with fake (meta) implementations, the way
the reference wraps its kernels as ``mylib::update_kv`` / ``mylib::decode``
(benchmark/blocktopk_decoder.py:23-58,171-184), so a layer built on them stays
traceable by ``torch.compile(fullgraph=True)``.
"""
from __future__ import annotations

import contextlib
from ctypes import c_void_p
from typing import Optional

import torch

from . import _lib

HEAD_DIM = 128
HEAD_DIMS = (64, 128)  # head dimensions the page path and the layer's row kernels are built for
PAGE_SIZE = 16


_EMPTY_STANDIN = {}


def _ptr(t: Optional[torch.Tensor]):
    """Device pointer of a tensor (None -> NULL).  An empty tensor has no storage
    and would read as NULL ("argument missing" to the C ABI); it is passed as a
    pointer to a small per-device buffer that nothing dereferences."""
    if t is None:
        return None
    if t.numel() == 0:
        buf = _EMPTY_STANDIN.get(t.device)
        if buf is None:
            buf = _EMPTY_STANDIN[t.device] = torch.zeros(64, dtype=torch.uint8, device=t.device)
        return c_void_p(buf.data_ptr())
    return c_void_p(t.data_ptr())


_NO_GUARD = contextlib.nullcontext()


def _on(device):
    """Context that makes ``device`` current for a launch; free when it already is."""
    idx = device.index
    if idx is None or idx == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(device)


def _stream(device) -> c_void_p:
    return c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _require(t: torch.Tensor, name: str, dtype: torch.dtype, ndim=None, device=None):
    # On the launch path of every call: the cheap tests first, messages built only on failure.
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
    if t.dtype is not dtype and (not isinstance(dtype, tuple) or t.dtype not in dtype):
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (device 'cuda'), got {t.device}")
    if device is not None and t.device != device:
        raise ValueError(f"{name} is on {t.device}, expected {device}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if ndim is not None:
        d = t.dim()
        if d != ndim and (not isinstance(ndim, tuple) or d not in ndim):
            raise ValueError(f"{name} must have {ndim} dimensions, got shape {tuple(t.shape)}")


# q, k, v, kv_cache, kbar and out hold bfloat16, or float16 (the reference's --dtype float16,
# benchmark/blocktopk.py:18): one dtype per call, which picks the kin_* or kin_*_f16 entry point
ELEM_DTYPES = (torch.bfloat16, torch.float16)


def _entry(lib, name: str, dtype: torch.dtype):
    return getattr(lib, name + "_f16" if dtype is torch.float16 else name)


def _cache_dims(kv_cache: torch.Tensor):
    _require(kv_cache, "kv_cache", ELEM_DTYPES, 5)
    num_pages, two, page_size, num_kv_heads, head_dim = kv_cache.shape
    if two != 2:
        raise ValueError(f"kv_cache must be [num_pages, 2, page_size, num_kv_heads, head_dim], got {tuple(kv_cache.shape)}")
    return num_pages, page_size, num_kv_heads, head_dim


def _kbar_pages(kbar: torch.Tensor, batch: int, num_kv_heads: int, head_dim: int, dtype: torch.dtype, slot_ids=None) -> int:
    """kbar is [B, Hkv, pages, D] (head-major), or the reference's [B, pages, D]
    when Hkv == 1 (the same bytes).  With ``slot_ids`` its first dimension counts
    cache slots, not sequences."""
    _require(kbar, "kbar", dtype, (3, 4))
    rows_ok = kbar.shape[0] == batch or (slot_ids is not None and kbar.shape[0] >= 1)
    if kbar.dim() == 3:
        ok = num_kv_heads == 1 and rows_ok and kbar.shape[2] == head_dim
        pages = kbar.shape[1]
    else:
        ok = rows_ok and kbar.shape[1] == num_kv_heads and kbar.shape[3] == head_dim
        pages = kbar.shape[2]
    if not ok:
        raise ValueError(
            f"kbar shape {tuple(kbar.shape)} does not match batch={batch}, num_kv_heads={num_kv_heads}, head_dim={head_dim} "
            "(expected [batch, num_kv_heads, pages, head_dim]; [slots, ...] with slot_ids)"
        )
    return pages


def _slots(slot_ids, kbar, batch: int, device):
    """(pointer, num_slots) of the optional ``slot_ids`` [batch] int32: sequence b's mean
    keys are ``kbar[slot_ids[b]]`` (the reference's kernels index the cache by slot and
    q, k, v, out by position in the active batch,
    LiteSys/litesys/attention/cache_utils.py:40-51,67-70)."""
    if slot_ids is None:
        return None, 0
    _require(slot_ids, "slot_ids", torch.int32, 1, device)
    if slot_ids.numel() != batch:
        raise ValueError(f"slot_ids must have batch={batch} entries, got {slot_ids.numel()}")
    return _ptr(slot_ids), (0 if kbar is None else kbar.shape[0])


def _table(page_indices, page_indptr, last_page_len, batch, device):
    _require(page_indices, "page_indices", torch.int32, 1, device)
    _require(page_indptr, "page_indptr", torch.int32, 1, device)
    if page_indptr.numel() != batch + 1:
        raise ValueError(f"page_indptr must have batch+1={batch + 1} entries, got {page_indptr.numel()}")
    if last_page_len is not None:
        _require(last_page_len, "last_page_len", torch.int32, 1, device)
        if last_page_len.numel() != batch:
            raise ValueError(f"last_page_len must have batch={batch} entries, got {last_page_len.numel()}")


# ---------------------------------------------------------------------------
# (1) append
# ---------------------------------------------------------------------------


def append_paged_kv(k, v, kv_cache, kbar, page_indices, page_indptr, last_page_len, slot_ids=None) -> None:
    """Write one new token per sequence into the paged cache (and refresh the
    mean key of a page that becomes full).  Stands in for ``mylib::update_kv``
    (benchmark/blocktopk_decoder.py:23-46,209-213).  The page table describes
    the cache after the append.  ``kbar`` may be None.  ``slot_ids`` (int32
    [batch], optional): ``kbar`` is laid out by cache slot and sequence b uses
    ``kbar[slot_ids[b]]``."""
    num_pages, page_size, num_kv_heads, head_dim = _cache_dims(kv_cache)
    dev = kv_cache.device
    dt = kv_cache.dtype
    _require(k, "k", dt, 3, dev)
    _require(v, "v", dt, 3, dev)
    batch = k.shape[0]
    if tuple(k.shape) != (batch, num_kv_heads, head_dim) or k.shape != v.shape:
        raise ValueError(f"k and v must be [batch, {num_kv_heads}, {head_dim}], got {tuple(k.shape)} and {tuple(v.shape)}")
    _table(page_indices, page_indptr, last_page_len, batch, dev)
    kbar_pages = 0
    if kbar is not None:
        kbar_pages = _kbar_pages(kbar, batch, num_kv_heads, head_dim, dt, slot_ids)
        if kbar.device != dev:
            raise ValueError("kbar must be on the same device as kv_cache")
    sp, ns = _slots(slot_ids, kbar, batch, dev)
    lib = _lib.load()
    with _on(dev):
        _lib.check(
            _entry(lib, "kin_append_paged_kv", dt)(
                _ptr(k), _ptr(v), _ptr(kv_cache), _ptr(kbar), _ptr(page_indices), _ptr(page_indptr),
                _ptr(last_page_len), batch, num_kv_heads, head_dim, page_size, num_pages, kbar_pages, sp, ns, _stream(dev),
            )
        )


def append_paged_kv_ragged(k, v, append_indptr, kv_cache, kbar, page_indices, page_indptr, last_page_len,
                           max_append_len: Optional[int] = None, slot_ids=None) -> None:
    """Write ``append_indptr[b+1] - append_indptr[b]`` new tokens per sequence
    (rows of ``k`` / ``v`` [nnz, num_kv_heads, head_dim]) into the paged cache and
    refresh the mean key of every page that becomes full: the general form of
    ``mylib::update_kv`` (benchmark/blocktopk_decoder.py:23-46) and the paged
    counterpart of LiteSys' prefill write (batch_cache.py:112-131).  The page
    table describes the cache after the append.  ``max_append_len`` bounds the
    longest append (default: nnz; it is checked, the cost does not depend on it)."""
    num_pages, page_size, num_kv_heads, head_dim = _cache_dims(kv_cache)
    dev = kv_cache.device
    dt = kv_cache.dtype
    _require(k, "k", dt, 3, dev)
    _require(v, "v", dt, 3, dev)
    nnz = k.shape[0]
    if tuple(k.shape) != (nnz, num_kv_heads, head_dim) or k.shape != v.shape:
        raise ValueError(f"k and v must be [nnz, {num_kv_heads}, {head_dim}], got {tuple(k.shape)} and {tuple(v.shape)}")
    _require(append_indptr, "append_indptr", torch.int32, 1, dev)
    batch = append_indptr.numel() - 1
    if batch < 0:
        raise ValueError("append_indptr must have batch+1 entries")
    _table(page_indices, page_indptr, last_page_len, batch, dev)
    kbar_pages = 0
    if kbar is not None:
        kbar_pages = _kbar_pages(kbar, batch, num_kv_heads, head_dim, dt, slot_ids)
        if kbar.device != dev:
            raise ValueError("kbar must be on the same device as kv_cache")
    sp, ns = _slots(slot_ids, kbar, batch, dev)
    lib = _lib.load()
    with _on(dev):
        _lib.check(
            _entry(lib, "kin_append_paged_kv_ragged", dt)(
                _ptr(k), _ptr(v), _ptr(append_indptr), _ptr(kv_cache), _ptr(kbar), _ptr(page_indices), _ptr(page_indptr),
                _ptr(last_page_len), batch, nnz, nnz if max_append_len is None else int(max_append_len), num_kv_heads,
                head_dim, page_size, num_pages, kbar_pages, sp, ns, _stream(dev),
            )
        )


def build_kbar(kv_cache, kbar, page_indices, page_indptr, last_page_len, slot_ids=None) -> None:
    """Fill ``kbar`` with the mean key of every full page (prefill-side producer
    of what the reference calls compressed_key_cache,
    benchmark/blocktopk_decoder.py:166-168)."""
    num_pages, page_size, num_kv_heads, head_dim = _cache_dims(kv_cache)
    dev = kv_cache.device
    batch = page_indptr.numel() - 1
    _table(page_indices, page_indptr, last_page_len, batch, dev)
    kbar_pages = _kbar_pages(kbar, batch, num_kv_heads, head_dim, kv_cache.dtype, slot_ids)
    sp, ns = _slots(slot_ids, kbar, batch, dev)
    lib = _lib.load()
    with _on(dev):
        _lib.check(
            _entry(lib, "kin_build_kbar", kv_cache.dtype)(
                _ptr(kv_cache), _ptr(kbar), _ptr(page_indices), _ptr(page_indptr), _ptr(last_page_len),
                batch, num_kv_heads, head_dim, page_size, num_pages, kbar_pages, sp, ns, _stream(dev),
            )
        )


# ---------------------------------------------------------------------------
# (2)+(3) score + select
# ---------------------------------------------------------------------------


def sel_list_capacity(topk: int, sink_pages: int = 0, local_tokens: int = 1) -> int:
    """Longest page list the selector writes: the stride ``sel_pages`` needs."""
    return int(_lib.load().kin_sel_list_capacity(int(topk), int(sink_pages), int(local_tokens)))


def block_score_topk(q, kbar, page_indices, page_indptr, last_page_len, topk, sel_pages, sel_count, sel_logical=None,
                     scores_out=None, sink_pages: int = 0, local_tokens: int = 1, workspace=None,
                     page_size: int = PAGE_SIZE, slot_ids=None) -> None:
    """Score every candidate page with the group-mean query and write the
    top-``topk`` pages plus the last page into ``sel_pages`` / ``sel_count``
    (in place: fixed buffers, as the reference registers with its decode
    wrapper, benchmark/blocktopk_decoder.py:143,156-159).  Stands in for
    lines 216-221 of that file.  The first ``sink_pages`` pages and the pages
    that hold the newest ``local_tokens`` tokens are always attended and never
    candidates (0 and 1 give the reference's "top-k plus the last page"; 1 and
    LiteSys' ``local`` on a cache stored 12 slots into its first page give
    LiteSys/litesys/attention/sparsity_utils.py:24-47).  List order: sink pages,
    selected pages by descending score, local pages.  ``workspace`` (uint8,
    ``step_workspace_bytes``; optional) lets few, long sequences spread their
    scoring over the GPU.  ``page_size``: tokens per page of the cache the table
    describes (16, 32, 64 or 128)."""
    _require(q, "q", ELEM_DTYPES, 3)
    dev = q.device
    batch, num_q_heads, head_dim = q.shape
    _require(sel_pages, "sel_pages", torch.int32, 3, dev)
    num_kv_heads, sel_stride = sel_pages.shape[1], sel_pages.shape[2]
    if sel_pages.shape[0] != batch:
        raise ValueError(f"sel_pages must be [batch, num_kv_heads, stride], got {tuple(sel_pages.shape)}")
    _require(sel_count, "sel_count", torch.int32, 2, dev)
    if tuple(sel_count.shape) != (batch, num_kv_heads):
        raise ValueError(f"sel_count must be [{batch}, {num_kv_heads}], got {tuple(sel_count.shape)}")
    kbar_pages = _kbar_pages(kbar, batch, num_kv_heads, head_dim, q.dtype, slot_ids)
    sp, ns = _slots(slot_ids, kbar, batch, dev)
    _table(page_indices, page_indptr, last_page_len, batch, dev)
    if last_page_len is None:
        raise TypeError("last_page_len is required")
    if sel_logical is not None:
        _require(sel_logical, "sel_logical", torch.int32, 3, dev)
        if tuple(sel_logical.shape) != (batch, num_kv_heads, topk):
            raise ValueError(f"sel_logical must be [{batch}, {num_kv_heads}, {topk}], got {tuple(sel_logical.shape)}")
    if scores_out is not None:
        _require(scores_out, "scores_out", torch.float32, 3, dev)
        if tuple(scores_out.shape) != (batch, num_kv_heads, kbar_pages):
            raise ValueError(f"scores_out must be [{batch}, {num_kv_heads}, {kbar_pages}], got {tuple(scores_out.shape)}")
    if workspace is not None:
        _require(workspace, "workspace", torch.uint8, 1, dev)
    lib = _lib.load()
    with _on(dev):
        _lib.check(
            _entry(lib, "kin_block_score_topk", q.dtype)(
                _ptr(q), _ptr(kbar), _ptr(page_indices), _ptr(page_indptr), _ptr(last_page_len), int(topk), int(sink_pages),
                int(local_tokens), _ptr(sel_pages), _ptr(sel_count), _ptr(sel_logical), _ptr(scores_out), batch, num_q_heads,
                num_kv_heads, head_dim, int(page_size), kbar_pages, sel_stride, _ptr(workspace),
                workspace.numel() if workspace is not None else 0, sp, ns, _stream(dev),
            )
        )


# ---------------------------------------------------------------------------
# (4) attention
# ---------------------------------------------------------------------------


def decode_workspace_bytes(batch, num_q_heads, num_kv_heads, max_pages_per_list, num_splits=0, head_dim=HEAD_DIM) -> int:
    return int(_lib.load().kin_decode_workspace_bytes(batch, num_q_heads, num_kv_heads, head_dim, max_pages_per_list, num_splits))


def step_workspace_bytes(batch: int, num_kv_heads: int, kbar_pages: int) -> int:
    """Bytes of workspace the fused step can use for this shape (0: none)."""
    return int(_lib.load().kin_step_workspace_bytes(int(batch), int(num_kv_heads), int(kbar_pages)))


def decode_auto_splits(batch, num_kv_heads, max_pages_per_list) -> int:
    return int(_lib.load().kin_decode_auto_splits(batch, num_kv_heads, max_pages_per_list))


def _decode_common(q, kv_cache, last_page_len, out, lse, workspace):
    num_pages, page_size, num_kv_heads, head_dim = _cache_dims(kv_cache)
    dev = kv_cache.device
    _require(q, "q", kv_cache.dtype, 3, dev)
    batch, num_q_heads, qd = q.shape
    if qd != head_dim:
        raise ValueError(f"q head_dim {qd} != kv_cache head_dim {head_dim}")
    _require(last_page_len, "last_page_len", torch.int32, 1, dev)
    if last_page_len.numel() != batch:
        raise ValueError(f"last_page_len must have batch={batch} entries, got {last_page_len.numel()}")
    if out is None:
        out = torch.empty_like(q)
    else:
        _require(out, "out", kv_cache.dtype, 3, dev)
        if out.shape != q.shape:
            raise ValueError(f"out shape {tuple(out.shape)} != q shape {tuple(q.shape)}")
    if lse is not None:
        _require(lse, "lse", torch.float32, 2, dev)
        if tuple(lse.shape) != (batch, num_q_heads):
            raise ValueError(f"lse must be [{batch}, {num_q_heads}], got {tuple(lse.shape)}")
    if workspace is not None:
        _require(workspace, "workspace", torch.uint8, 1, dev)
    return dev, batch, num_q_heads, num_kv_heads, head_dim, page_size, num_pages, out


def _workspace(workspace, dev, batch, hq, hkv, max_pages, num_splits):
    """The caller's workspace, or a fresh one when none was given and the split
    count needs it (like ``out``: allocated here only as a convenience; loops
    that must not allocate pass both)."""
    if workspace is None:
        need = decode_workspace_bytes(batch, hq, hkv, max_pages, num_splits)
        if need:
            workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    return workspace, (0 if workspace is None else workspace.numel())


def sparse_paged_decode(q, kv_cache, sel_pages, sel_count, last_page_len, out=None, lse=None, workspace=None,
                        sm_scale: float = 0.0, num_splits: int = 0, first_page_offset: int = 0):
    """Attention of one query token per sequence over the listed pages; stands
    in for ``mylib::decode`` (benchmark/blocktopk_decoder.py:171-184,223-225).
    ``first_page_offset`` leading token slots of each list's first page are
    padding.  Returns ``out`` [batch, num_q_heads, head_dim] bf16."""
    dev, batch, hq, hkv, d, ps, num_pages, out = _decode_common(q, kv_cache, last_page_len, out, lse, workspace)
    _require(sel_pages, "sel_pages", torch.int32, 3, dev)
    _require(sel_count, "sel_count", torch.int32, 2, dev)
    if sel_pages.shape[:2] != (batch, hkv) or tuple(sel_count.shape) != (batch, hkv):
        raise ValueError(
            f"sel_pages/sel_count must be [{batch}, {hkv}, stride] / [{batch}, {hkv}], got {tuple(sel_pages.shape)} / {tuple(sel_count.shape)}"
        )
    workspace, ws_bytes = _workspace(workspace, dev, batch, hq, hkv, sel_pages.shape[2], int(num_splits))
    lib = _lib.load()
    with _on(dev):
        _lib.check(
            _entry(lib, "kin_sparse_paged_decode", kv_cache.dtype)(
                _ptr(q), _ptr(kv_cache), _ptr(sel_pages), _ptr(sel_count), _ptr(last_page_len), _ptr(out), _ptr(lse),
                _ptr(workspace), ws_bytes, batch, hq, hkv, d, ps, num_pages, sel_pages.shape[2], int(first_page_offset),
                float(sm_scale), int(num_splits), _stream(dev),
            )
        )
    return out


def dense_paged_decode(q, kv_cache, page_indices, page_indptr, last_page_len, max_pages_per_seq, out=None, lse=None,
                       workspace=None, sm_scale: float = 0.0, num_splits: int = 0, first_page_offset: int = 0):
    """Attention over every page of each sequence; the dense baseline
    (benchmark/dense_decoder.py:149-170,211-219)."""
    dev, batch, hq, hkv, d, ps, num_pages, out = _decode_common(q, kv_cache, last_page_len, out, lse, workspace)
    _table(page_indices, page_indptr, None, batch, dev)
    workspace, ws_bytes = _workspace(workspace, dev, batch, hq, hkv, int(max_pages_per_seq), int(num_splits))
    lib = _lib.load()
    with _on(dev):
        _lib.check(
            _entry(lib, "kin_dense_paged_decode", kv_cache.dtype)(
                _ptr(q), _ptr(kv_cache), _ptr(page_indices), _ptr(page_indptr), _ptr(last_page_len), _ptr(out),
                _ptr(lse), _ptr(workspace), ws_bytes, batch, hq, hkv, d, ps, num_pages, int(max_pages_per_seq),
                int(first_page_offset), float(sm_scale), int(num_splits), _stream(dev),
            )
        )
    return out


def prefer_fused_step(batch: int, num_kv_heads: int, max_pages_per_seq: int, topk: int) -> bool:
    """Which of the two equivalent decode-step paths to use.  The single-launch
    kernel saves two dependent dispatches, the selector's drain and the attention
    ramp-up; given its workspace it shares a list between workgroups when the lists
    are few (split attention up to 128 lists, split scoring for very long
    sequences).  Measured on MI355X against the three launches queued back to back
    (fused / three): 1..128 lists of 2049 pages, k = 128..2048: 0.84..1.04; of 257
    pages: 0.5; 8..32 lists of 4097..8193 pages: k = 128 0.96..1.02, k = 256..512
    1.1..1.3, k = 2048 1.13 (scoring a whole list in every part costs as much as
    the parts save); 200..256 lists
    0.95..0.98; 260..300 lists k <= 768 0.96..0.98, k = 1024 1.17..1.20 (some CUs hold
    two long lists, the others one); 350 lists and more 0.96..1.00.  Hence: fused,
    except few lists of more than 4096 pages with k >= 256, and 257..349 lists with
    k > 768."""
    lists = batch * num_kv_heads
    if lists < 160:
        return not (max_pages_per_seq > 4096 and topk >= 256)
    if 256 < lists < 350:
        return topk <= 768
    return True


def blocktopk_decode_step(q, k, v, kv_cache, kbar, page_indices, page_indptr, last_page_len, topk, out=None, lse=None,
                          sel_pages=None, sel_count=None, sm_scale: float = 0.0, sink_pages: int = 0,
                          local_tokens: int = 1, first_page_offset: int = 0, workspace=None, static_scratch: bool = False,
                          slot_ids=None, slot_lens=None):
    """append -> score -> select -> attend in one launch: lines 209-225 of the
    reference layer's forward (benchmark/blocktopk_decoder.py) as a single
    kernel.  ``k``/``v`` may be None (no append); ``sel_pages``/``sel_count`` are
    optional outputs.  ``workspace`` (``step_workspace_bytes``; allocated here when
    None and the shape profits) lets several workgroups share a list when the lists
    are few: split attention, or split scoring for very long sequences.  ``static_scratch=True`` calls ``kin_blocktopk_decode_step_static``
    instead: the library's built-in device array is the workspace and nothing is
    allocated (``out`` must then be given; ``workspace`` must be None).  ``slot_ids``: ``kbar`` is laid
    out by cache slot; ``slot_lens`` (int32, one entry per row block of ``kbar``): a token counter
    per slot that the kernel advances by one for every sequence it appends to.
    Returns ``out`` [batch, num_q_heads, head_dim] bf16."""
    if static_scratch and (out is None or workspace is not None):
        raise ValueError("static_scratch=True needs a caller-provided out and takes no workspace")
    dev, batch, hq, hkv, d, ps, num_pages, out = _decode_common(q, kv_cache, last_page_len, out, lse, workspace)
    _table(page_indices, page_indptr, last_page_len, batch, dev)
    dt = kv_cache.dtype
    kbar_pages = _kbar_pages(kbar, batch, hkv, d, dt, slot_ids)
    sp, ns = _slots(slot_ids, kbar, batch, dev)
    if slot_lens is not None:
        _require(slot_lens, "slot_lens", torch.int32, 1, dev)
        if slot_lens.numel() != kbar.shape[0]:
            raise ValueError(f"slot_lens must have one entry per row block of kbar ({kbar.shape[0]}), got {slot_lens.numel()}")
    if (k is None) != (v is None):
        raise ValueError("k and v must both be given or both be None")
    if k is not None:
        _require(k, "k", dt, 3, dev)
        _require(v, "v", dt, 3, dev)
        if tuple(k.shape) != (batch, hkv, d) or k.shape != v.shape:
            raise ValueError(f"k and v must be [{batch}, {hkv}, {d}], got {tuple(k.shape)} and {tuple(v.shape)}")
    sel_stride = 0
    if (sel_pages is None) != (sel_count is None):
        raise ValueError("sel_pages and sel_count must both be given or both be None")
    if sel_pages is not None:
        _require(sel_pages, "sel_pages", torch.int32, 3, dev)
        _require(sel_count, "sel_count", torch.int32, 2, dev)
        if sel_pages.shape[:2] != (batch, hkv) or tuple(sel_count.shape) != (batch, hkv):
            raise ValueError(f"sel_pages/sel_count must be [{batch}, {hkv}, stride] / [{batch}, {hkv}]")
        sel_stride = sel_pages.shape[2]
    lib = _lib.load()
    if static_scratch:
        if dt is not torch.bfloat16:
            raise ValueError("static_scratch=True is built for bfloat16 only")
        with _on(dev):
            _lib.check(
                lib.kin_blocktopk_decode_step_static(
                    _ptr(q), _ptr(k), _ptr(v), _ptr(kv_cache), _ptr(kbar), _ptr(page_indices), _ptr(page_indptr),
                    _ptr(last_page_len), int(topk), int(sink_pages), int(local_tokens), _ptr(sel_pages), _ptr(sel_count),
                    _ptr(out), _ptr(lse), batch, hq, hkv, d, ps, num_pages, kbar_pages, sel_stride, int(first_page_offset),
                    float(sm_scale), sp, ns, _ptr(slot_lens), _stream(dev),
                )
            )
        return out
    if workspace is None:
        need = step_workspace_bytes(batch, hkv, kbar_pages)
        if need:
            workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    with _on(dev):
        _lib.check(
            _entry(lib, "kin_blocktopk_decode_step", dt)(
                _ptr(q), _ptr(k), _ptr(v), _ptr(kv_cache), _ptr(kbar), _ptr(page_indices), _ptr(page_indptr),
                _ptr(last_page_len), int(topk), int(sink_pages), int(local_tokens), _ptr(sel_pages), _ptr(sel_count),
                _ptr(out), _ptr(lse), batch, hq, hkv, d, ps, num_pages, kbar_pages, sel_stride, int(first_page_offset),
                float(sm_scale), _ptr(workspace), 0 if workspace is None else workspace.numel(), sp, ns, _ptr(slot_lens),
                _stream(dev),
            )
        )
    return out


class DecodeStepPlan:
    """``blocktopk_decode_step`` with everything but q, k, v and out checked and bound once, for
    callers that make the same call again and again on buffers they own (a KV manager: every layer
    of every decode step).  The tensors given here must stay alive and in place; a call checks only
    the four tensors it is given and hands their pointers to the C ABI (a few microseconds of host
    time instead of ~20)."""

    def __init__(self, kv_cache, kbar, page_indices, page_indptr, last_page_len, topk: int, num_q_heads: int,
                 sm_scale: float = 0.0, sink_pages: int = 0, local_tokens: int = 1, first_page_offset: int = 0,
                 workspace=None, slot_ids=None, slot_lens=None):
        num_pages, page_size, hkv, d = _cache_dims(kv_cache)
        dev, dt = kv_cache.device, kv_cache.dtype
        batch = page_indptr.numel() - 1
        _table(page_indices, page_indptr, last_page_len, batch, dev)
        kbar_pages = _kbar_pages(kbar, batch, hkv, d, dt, slot_ids)
        sp, ns = _slots(slot_ids, kbar, batch, dev)
        if workspace is not None:
            _require(workspace, "workspace", torch.uint8, 1, dev)
        if num_q_heads % hkv:
            raise ValueError(f"num_q_heads={num_q_heads} is not a multiple of num_kv_heads={hkv}")
        if slot_lens is not None:
            _require(slot_lens, "slot_lens", torch.int32, 1, dev)
            if slot_lens.numel() != kbar.shape[0]:
                raise ValueError("slot_lens must have one entry per row block of kbar")
        self._keep = (kv_cache, kbar, page_indices, page_indptr, last_page_len, workspace, slot_ids, slot_lens)
        self._fn = _entry(_lib.load(), "kin_blocktopk_decode_step", dt)
        self._dev, self._dt = dev, dt
        self._q_shape, self._k_shape = (batch, int(num_q_heads), d), (batch, hkv, d)
        self._head = (_ptr(kv_cache), _ptr(kbar), _ptr(page_indices), _ptr(page_indptr), _ptr(last_page_len), int(topk),
                      int(sink_pages), int(local_tokens), None, None)
        self._tail = (batch, int(num_q_heads), hkv, d, page_size, num_pages, kbar_pages, 0, int(first_page_offset), float(sm_scale),
                      _ptr(workspace), 0 if workspace is None else workspace.numel(), sp, ns, _ptr(slot_lens))

    def __call__(self, q, k, v, out):
        for t, shape in ((q, self._q_shape), (k, self._k_shape), (v, self._k_shape), (out, self._q_shape)):
            if t.dtype is not self._dt or t.device != self._dev or tuple(t.shape) != shape or not t.is_contiguous():
                raise ValueError(f"DecodeStepPlan: expected a contiguous {self._dt} tensor of shape {shape} on {self._dev}, "
                                 f"got {t.dtype} {tuple(t.shape)} on {t.device}")
        with _on(self._dev):
            _lib.check(self._fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), *self._head, out.data_ptr(), None, *self._tail,
                                _stream(self._dev)))
        return out


def token_topk_workspace_bytes(batch: int, num_kv_heads: int, max_pages_per_seq: int) -> int:
    return int(_lib.load().kin_token_topk_workspace_bytes(int(batch), int(num_kv_heads), int(max_pages_per_seq)))


def _token_policy(q, kv_cache, page_indices, page_indptr, last_page_len, out, lse, sel_tokens, sel_count, workspace,
                  need_bytes):
    dev, batch, hq, hkv, d, ps, num_pages, out = _decode_common(q, kv_cache, last_page_len, out, lse, None)
    _table(page_indices, page_indptr, last_page_len, batch, dev)
    sel_stride = 0
    if (sel_tokens is None) != (sel_count is None):
        raise ValueError("sel_tokens and sel_count must both be given or both be None")
    if sel_tokens is not None:
        _require(sel_tokens, "sel_tokens", torch.int32, 3, dev)
        _require(sel_count, "sel_count", torch.int32, 2, dev)
        if sel_tokens.shape[:2] != (batch, hkv) or tuple(sel_count.shape) != (batch, hkv):
            raise ValueError(f"sel_tokens/sel_count must be [{batch}, {hkv}, stride] / [{batch}, {hkv}]")
        sel_stride = sel_tokens.shape[2]
    if workspace is None:
        workspace = torch.empty(max(need_bytes(batch, hkv), 16), dtype=torch.uint8, device=dev)
    else:
        _require(workspace, "workspace", torch.uint8, 1, dev)
    return dev, batch, hq, hkv, d, ps, num_pages, out, sel_stride, workspace


def token_topk_decode(q, kv_cache, page_indices, page_indptr, last_page_len, topk_tokens: int, max_pages_per_seq: int,
                      sink_tokens: int = 4, local_tokens: int = 1, first_page_offset: int = 0, out=None, lse=None,
                      sel_tokens=None, sel_count=None, workspace=None, sm_scale: float = 0.0):
    """Token-level top-k sparse decode attention: LiteSys' ``topk_sparsity``
    (LiteSys/litesys/attention/sparsity_utils.py:6-21) inside its decode
    (batch_cache.py:154-168) in one launch on the paged cache.  The first
    ``sink_tokens`` and newest ``local_tokens`` tokens are always attended; of
    the rest, the ``topk_tokens`` with the largest group-mean logit per KV
    head.  The new token must already be appended.  Returns ``out``."""
    dev, batch, hq, hkv, d, ps, num_pages, out, sel_stride, workspace = _token_policy(
        q, kv_cache, page_indices, page_indptr, last_page_len, out, lse, sel_tokens, sel_count, workspace,
        lambda b, h: token_topk_workspace_bytes(b, h, max_pages_per_seq))
    lib = _lib.load()
    with _on(dev):
        _lib.check(
            _entry(lib, "kin_token_topk_decode", kv_cache.dtype)(
                _ptr(q), _ptr(kv_cache), _ptr(page_indices), _ptr(page_indptr), _ptr(last_page_len), int(topk_tokens),
                int(sink_tokens), int(local_tokens), int(first_page_offset), _ptr(sel_tokens), _ptr(sel_count), _ptr(out),
                _ptr(lse), _ptr(workspace), workspace.numel(), batch, hq, hkv, d, ps, num_pages, int(max_pages_per_seq),
                sel_stride, float(sm_scale), _stream(dev),
            )
        )
    return out


def strided_topk_workspace_bytes(batch: int, num_kv_heads: int, max_pages_per_seq: int) -> int:
    return int(_lib.load().kin_strided_topk_workspace_bytes(int(batch), int(num_kv_heads), int(max_pages_per_seq)))


def strided_topk_decode(q, kv_cache, page_indices, page_indptr, last_page_len, topk_blocks: int, max_pages_per_seq: int,
                        block_size: int = 16, stride: int = 8, sink_tokens: int = 4, local_tokens: int = 1,
                        first_page_offset: int = 0, out=None, lse=None, sel_tokens=None, sel_count=None, workspace=None,
                        sm_scale: float = 0.0):
    """Strided overlapping-block top-k sparse decode attention: LiteSys'
    ``strided_blockwise_topk_sparsity`` (sparsity_utils.py:49-105) inside its
    decode, in one launch on the paged cache.  Blocks of ``block_size`` candidate
    tokens start every ``stride`` tokens; the ``2 * topk_blocks`` best by mean
    logit are united and the ``topk_blocks * block_size`` lowest-positioned of
    their tokens attended, with the sink and local tokens.  Returns ``out``."""
    dev, batch, hq, hkv, d, ps, num_pages, out, sel_stride, workspace = _token_policy(
        q, kv_cache, page_indices, page_indptr, last_page_len, out, lse, sel_tokens, sel_count, workspace,
        lambda b, h: strided_topk_workspace_bytes(b, h, max_pages_per_seq))
    lib = _lib.load()
    with _on(dev):
        _lib.check(
            _entry(lib, "kin_strided_topk_decode", kv_cache.dtype)(
                _ptr(q), _ptr(kv_cache), _ptr(page_indices), _ptr(page_indptr), _ptr(last_page_len), int(topk_blocks),
                int(block_size), int(stride), int(sink_tokens), int(local_tokens), int(first_page_offset),
                _ptr(sel_tokens), _ptr(sel_count), _ptr(out), _ptr(lse), _ptr(workspace), workspace.numel(), batch, hq,
                hkv, d, ps, num_pages, int(max_pages_per_seq), sel_stride, float(sm_scale), _stream(dev),
            )
        )
    return out


def build_slot_page_table(seq_lens, pages_per_slot, page_size, page_indices, page_indptr, last_page_len, slot_ids=None) -> None:
    """CSR page table for a cache where slot ``s`` owns pages
    ``s*pages_per_slot ...`` (the paged stand-in for LiteSys' contiguous
    per-slot caches, LiteSys/litesys/attention/batch_cache.py:40-62).  Fills the
    three output tensors in place from the token counts ``seq_lens``."""
    _require(seq_lens, "seq_lens", torch.int32, 1)
    dev = seq_lens.device
    batch = seq_lens.numel()
    _require(page_indices, "page_indices", torch.int32, 1, dev)
    _require(page_indptr, "page_indptr", torch.int32, 1, dev)
    _require(last_page_len, "last_page_len", torch.int32, 1, dev)
    if page_indptr.numel() != batch + 1 or last_page_len.numel() != batch:
        raise ValueError("page_indptr needs batch+1 entries and last_page_len batch entries")
    if page_indices.numel() < batch * pages_per_slot:
        raise ValueError(f"page_indices needs room for batch*pages_per_slot = {batch * pages_per_slot} entries")
    if slot_ids is not None:
        _require(slot_ids, "slot_ids", torch.int32, 1, dev)
        if slot_ids.numel() != batch:
            raise ValueError("slot_ids must have one entry per sequence")
    lib = _lib.load()
    with _on(dev):
        _lib.check(
            lib.kin_build_slot_page_table(_ptr(slot_ids), _ptr(seq_lens), batch, int(pages_per_slot), int(page_size),
                                          _ptr(page_indices), _ptr(page_indptr), _ptr(last_page_len), _stream(dev))
        )


class PagePool:
    """Device-resident free list from which the slots of a slot-based cache draw
    their pages (kin_page_pool_*): the paged answer to LiteSys' fixed
    [max_batch, H_kv, max_len, D] caches and zeroing clear_cache
    (LiteSys/litesys/attention/batch_cache.py:40-62,147-152).  The pool may hold
    fewer pages than ``max_slots * pages_per_slot``; a finished slot returns its
    pages.  No method synchronises except ``status()`` / ``raise_on_overflow()``."""

    EXHAUSTED, SLOT_TOO_LONG, BAD_SLOT = 1, 2, 4

    def __init__(self, num_pool_pages: int, max_slots: int, pages_per_slot: int, page_size: int, device):
        self.num_pool_pages, self.max_slots = int(num_pool_pages), int(max_slots)
        self.pages_per_slot, self.page_size = int(pages_per_slot), int(page_size)
        self.free_stack = torch.empty(self.num_pool_pages, dtype=torch.int32, device=torch.device(device))
        self.device = dev = self.free_stack.device   # with its index, as tensors report it
        self.pool_state = torch.empty(2, dtype=torch.int32, device=dev)
        self.slot_table = torch.full((self.max_slots, self.pages_per_slot), -1, dtype=torch.int32, device=dev)
        self.slot_npages = torch.empty(self.max_slots, dtype=torch.int32, device=dev)
        with _on(dev):
            _lib.check(_lib.load().kin_page_pool_init(_ptr(self.free_stack), _ptr(self.pool_state), _ptr(self.slot_npages),
                                                      self.num_pool_pages, self.max_slots, _stream(dev)))

    def _lens(self, seq_lens, slot_ids):
        _require(seq_lens, "seq_lens", torch.int32, 1, self.device)
        if slot_ids is not None:
            _require(slot_ids, "slot_ids", torch.int32, 1, self.device)
            if slot_ids.numel() != seq_lens.numel():
                raise ValueError("slot_ids must have one entry per sequence")
        elif seq_lens.numel() > self.max_slots:
            raise ValueError(f"{seq_lens.numel()} sequences but only {self.max_slots} slots")
        return seq_lens.numel()

    def reserve(self, seq_lens, slot_ids=None) -> None:
        """Grow the slots to cover ``seq_lens`` tokens each (never shrinks; all or nothing)."""
        batch = self._lens(seq_lens, slot_ids)
        with _on(self.device):
            _lib.check(_lib.load().kin_page_pool_reserve(
                _ptr(slot_ids), _ptr(seq_lens), batch, self.pages_per_slot, self.page_size, _ptr(self.slot_table),
                _ptr(self.slot_npages), _ptr(self.free_stack), _ptr(self.pool_state), self.max_slots, _stream(self.device)))

    def release(self, slot_ids) -> None:
        """Return every page of the listed slots (int32 tensor of slot ids) to the pool."""
        _require(slot_ids, "slot_ids", torch.int32, 1, self.device)
        with _on(self.device):
            _lib.check(_lib.load().kin_page_pool_release(
                _ptr(slot_ids), slot_ids.numel(), self.pages_per_slot, _ptr(self.slot_table), _ptr(self.slot_npages),
                _ptr(self.free_stack), _ptr(self.pool_state), self.num_pool_pages, self.max_slots, _stream(self.device)))

    def build_page_table(self, seq_lens, page_indices, page_indptr, last_page_len, slot_ids=None) -> None:
        """CSR page table of the sequences from the slots' page lists (kin_build_pool_page_table)."""
        batch = self._lens(seq_lens, slot_ids)
        dev = self.device
        _require(page_indices, "page_indices", torch.int32, 1, dev)
        _require(page_indptr, "page_indptr", torch.int32, 1, dev)
        _require(last_page_len, "last_page_len", torch.int32, 1, dev)
        if page_indptr.numel() != batch + 1 or last_page_len.numel() != batch:
            raise ValueError("page_indptr needs batch+1 entries and last_page_len batch entries")
        if page_indices.numel() < min(batch * self.pages_per_slot, self.num_pool_pages):
            raise ValueError("page_indices needs room for min(batch*pages_per_slot, num_pool_pages) entries")
        with _on(dev):
            _lib.check(_lib.load().kin_build_pool_page_table(
                _ptr(slot_ids), _ptr(seq_lens), batch, self.pages_per_slot, self.page_size, _ptr(self.slot_table),
                _ptr(self.slot_npages), _ptr(page_indices), _ptr(page_indptr), _ptr(last_page_len), self.max_slots,
                _stream(dev)))

    def status(self):
        """(free pages, status bits) -- copies two ints to the host (synchronises)."""
        free, bits = self.pool_state.tolist()
        return free, bits

    def acknowledge(self) -> None:
        """Clear the status bits (the condition has been seen and dealt with)."""
        self.pool_state[1:2].zero_()

    def raise_on_overflow(self) -> None:
        """Raise if any earlier call ran out of pages, met a sequence longer than a slot can
        hold, or was given a slot id it could not use (synchronises; the kernels themselves
        cannot raise).  The bits are cleared first: the condition is reported once."""
        free, bits = self.status()
        if not bits:
            return
        self.acknowledge()
        if bits & self.EXHAUSTED:
            raise _lib.KineticsError(f"page pool exhausted: a reserve wanted more than the {free} free pages "
                                     f"(pool of {self.num_pool_pages}); the sequences it could not serve have an empty "
                                     "page list (nothing was written for them, their output is zero)")
        if bits & self.SLOT_TOO_LONG:
            raise ValueError(f"a sequence exceeds {self.pages_per_slot} pages of {self.page_size} tokens (max_seq_len); "
                             "it has an empty page list (nothing was written for it, its output is zero)")
        raise ValueError(f"a slot id outside [0, {self.max_slots}) or listed twice in one call was skipped")


def check_page_table(page_indices, page_indptr, last_page_len, page_size, num_pages) -> None:
    """Synchronous device-side validation of a page table (debugging aid);
    raises KineticsError on an invalid entry."""
    _require(page_indices, "page_indices", torch.int32, 1)
    dev = page_indices.device
    batch = page_indptr.numel() - 1
    _table(page_indices, page_indptr, last_page_len, batch, dev)
    scratch = torch.zeros(1, dtype=torch.int32, device=dev)
    lib = _lib.load()
    with _on(dev):
        _lib.check(
            lib.kin_check_page_table(
                _ptr(page_indices), _ptr(page_indptr), _ptr(last_page_len), batch, int(page_size), int(num_pages),
                page_indices.numel(), _ptr(scratch), _stream(dev),
            )
        )


# ---------------------------------------------------------------------------
# Row-wise layer kernels around the attention path
# ---------------------------------------------------------------------------

ACTIVATIONS = {"silu": 0, "gelu": 1, "relu": 2}


def _row_view(t: torch.Tensor, name: str, device=None, dtype=None):
    """(rows, width, row stride in elements) of a bf16 / fp16 tensor (``dtype``: that
    very type) whose rows are its last dimension: any contiguous shape, or a 2-D view
    with a row stride (a slice of a wider projection)."""
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
    if t.dtype not in ELEM_DTYPES or (dtype is not None and t.dtype != dtype):
        want = dtype if dtype is not None else "torch.bfloat16 or torch.float16"
        raise TypeError(f"{name} must be {want}, got {t.dtype}")
    if t.device.type != "cuda":
        raise ValueError(f"{name} must live on the GPU (device 'cuda'), got {t.device}")
    if device is not None and t.device != device:
        raise ValueError(f"{name} is on {t.device}, expected {device}")
    if t.dim() < 1:
        raise ValueError(f"{name} must have at least one dimension")
    width = t.shape[-1]
    if t.is_contiguous():
        return t.numel() // max(width, 1), width, width
    if t.dim() == 2 and t.stride(1) == 1:
        return t.shape[0], width, t.stride(0)
    raise ValueError(f"{name} must be contiguous, or 2-D with unit stride along its rows")


def rms_norm(x, weight, eps: float, residual=None, out=None) -> torch.Tensor:
    """RMSNorm over the last dimension with fp32 statistics: what the reference's
    ``layer_norm`` and ``qk_norm`` ops compute through flashinfer.rmsnorm
    (benchmark/model_utils.py:4-25).  With ``residual`` (contiguous, same shape)
    the add in front of the norm is folded in as in ``fused_layer_norm``
    (benchmark/model_utils.py:27-41): ``residual`` becomes ``x + residual`` and
    the norm of that sum is returned."""
    rows, hidden, x_stride = _row_view(x, "x")
    dev, dt = x.device, x.dtype
    _require(weight, "weight", dt, 1, dev)
    if weight.numel() != hidden:
        raise ValueError(f"weight has {weight.numel()} entries for rows of {hidden}")
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype, device=dev)
    orows, owidth, out_stride = _row_view(out, "out", dev, dt)
    if (orows, owidth) != (rows, hidden):
        raise ValueError(f"out shape {tuple(out.shape)} does not match x {tuple(x.shape)}")
    if residual is not None:
        _require(residual, "residual", dt, None, dev)
        if residual.numel() != rows * hidden or residual.shape[-1] != hidden:
            raise ValueError(f"residual shape {tuple(residual.shape)} does not match x {tuple(x.shape)}")
    lib = _lib.load()
    with _on(dev):
        _lib.check(_entry(lib, "kin_rms_norm", dt)(_ptr(x), _ptr(residual), _ptr(weight), _ptr(out), rows, hidden, x_stride,
                                                   out_stride, float(eps), _stream(dev)))
    return out


def qkv_norm_split(qkv, q_weight, k_weight, eps: float, num_q_heads: int, num_kv_heads: int):
    """From the fused projection ``qkv[batch, (Hq + 2*Hkv) * D]`` to contiguous
    ``q[batch, Hq, D]``, ``k[batch, Hkv, D]``, ``v[batch, Hkv, D]`` with the
    q and k heads RMS-normalised: the split, qk_norm calls and reshapes of
    benchmark/blocktopk_decoder.py:196-207 in one pass.  The head dimension D is the
    length of the norm weights (128 or 64)."""
    batch, width, stride = _row_view(qkv, "qkv")
    dev, dt = qkv.device, qkv.dtype
    _require(q_weight, "q_weight", dt, 1, dev)
    _require(k_weight, "k_weight", dt, 1, dev)
    head_dim = q_weight.numel()
    if head_dim not in HEAD_DIMS or k_weight.numel() != head_dim:
        raise ValueError(f"q_weight and k_weight must have the same number of entries, one of {HEAD_DIMS}; "
                         f"got {q_weight.numel()} and {k_weight.numel()}")
    if width != (num_q_heads + 2 * num_kv_heads) * head_dim:
        raise ValueError(f"qkv rows have {width} elements, expected (Hq + 2*Hkv) * {head_dim} = "
                         f"{(num_q_heads + 2 * num_kv_heads) * head_dim}")
    q = torch.empty(batch, num_q_heads, head_dim, dtype=dt, device=dev)
    k = torch.empty(batch, num_kv_heads, head_dim, dtype=dt, device=dev)
    v = torch.empty(batch, num_kv_heads, head_dim, dtype=dt, device=dev)
    lib = _lib.load()
    with _on(dev):
        _lib.check(_entry(lib, "kin_qkv_norm_split", dt)(_ptr(qkv), stride, _ptr(q_weight), _ptr(k_weight), float(eps),
                                                         _ptr(q), _ptr(k), _ptr(v), batch, int(num_q_heads),
                                                         int(num_kv_heads), head_dim, _stream(dev)))
    return q, k, v


def gated_act(gate, up, act: str = "silu", out=None) -> torch.Tensor:
    """``act(gate) * up`` of the gated MLP (benchmark/blocktopk_decoder.py:234-237),
    rounded to bf16 after the activation and after the product as the two tensor
    operations round (bf16 or fp16, whichever the tensors are).  ``gate`` and ``up`` may be column slices of one fused
    projection (2-D views with a row stride)."""
    if act not in ACTIVATIONS:
        raise ValueError(f"act must be one of {sorted(ACTIVATIONS)}, got {act!r}")
    rows, inter, g_stride = _row_view(gate, "gate")
    dev, dt = gate.device, gate.dtype
    urows, uwidth, u_stride = _row_view(up, "up", dev, dt)
    if (urows, uwidth) != (rows, inter):
        raise ValueError(f"up shape {tuple(up.shape)} does not match gate {tuple(gate.shape)}")
    if out is None:
        out = torch.empty(gate.shape, dtype=dt, device=dev)
    _require(out, "out", dt, None, dev)
    if out.numel() != rows * inter or out.shape[-1] != inter:
        raise ValueError(f"out shape {tuple(out.shape)} does not match gate {tuple(gate.shape)}")
    lib = _lib.load()
    with _on(dev):
        _lib.check(_entry(lib, "kin_gated_act", dt)(_ptr(gate), _ptr(up), _ptr(out), rows, inter, g_stride, u_stride,
                                                    ACTIVATIONS[act], _stream(dev)))
    return out


# ---------------------------------------------------------------------------
# torch.library registration (namespace "kinetics", defined once at import)
# ---------------------------------------------------------------------------

torch.library.define(
    "kinetics::append_paged_kv",
    "(Tensor k, Tensor v, Tensor(a!) kv_cache, Tensor(b!)? kbar, Tensor page_indices, Tensor page_indptr, "
    "Tensor last_page_len, Tensor? slot_ids=None) -> ()",
)
# Same argument order as the reference's mylib::update_kv
# (benchmark/blocktopk_decoder.py:23-26), plus the mean-key cache it has to keep current.
torch.library.define(
    "kinetics::update_kv",
    "(Tensor k, Tensor v, Tensor kv_append_indptr, Tensor(a!) kv_cache, Tensor kv_page_indices, Tensor kv_page_indptr, "
    "Tensor cachelen, Tensor(b!)? kbar=None, Tensor? slot_ids=None) -> ()",
)
torch.library.define(
    "kinetics::block_score_topk",
    "(Tensor q, Tensor kbar, Tensor page_indices, Tensor page_indptr, Tensor last_page_len, int topk, "
    "Tensor(a!) sel_pages, Tensor(b!) sel_count, int sink_pages=0, int local_tokens=1, Tensor(c!)? workspace=None, "
    "int page_size=16, Tensor? slot_ids=None) -> ()",
)
torch.library.define(
    "kinetics::sparse_paged_decode",
    "(Tensor q, Tensor kv_cache, Tensor sel_pages, Tensor sel_count, Tensor last_page_len, Tensor(a!)? workspace, "
    "float sm_scale, int num_splits, int first_page_offset=0) -> Tensor",
)
torch.library.define(
    "kinetics::dense_paged_decode",
    "(Tensor q, Tensor kv_cache, Tensor page_indices, Tensor page_indptr, Tensor last_page_len, "
    "int max_pages_per_seq, Tensor(a!)? workspace, float sm_scale, int num_splits, int first_page_offset=0) -> Tensor",
)


torch.library.define(
    "kinetics::token_topk_decode",
    "(Tensor q, Tensor kv_cache, Tensor page_indices, Tensor page_indptr, Tensor last_page_len, int topk_tokens, "
    "int max_pages_per_seq, int sink_tokens, int local_tokens, int first_page_offset, Tensor(a!) workspace, "
    "float sm_scale) -> Tensor",
)


@torch.library.impl("kinetics::token_topk_decode", "cuda")
def _token_impl(q, kv_cache, page_indices, page_indptr, last_page_len, topk_tokens, max_pages_per_seq, sink_tokens,
                local_tokens, first_page_offset, workspace, sm_scale):
    return token_topk_decode(q, kv_cache, page_indices, page_indptr, last_page_len, topk_tokens, max_pages_per_seq,
                             sink_tokens=sink_tokens, local_tokens=local_tokens, first_page_offset=first_page_offset,
                             workspace=workspace, sm_scale=sm_scale)


@torch.library.register_fake("kinetics::token_topk_decode")
def _token_fake(q, kv_cache, page_indices, page_indptr, last_page_len, topk_tokens, max_pages_per_seq, sink_tokens,
                local_tokens, first_page_offset, workspace, sm_scale):
    return torch.empty_like(q)


torch.library.define(
    "kinetics::blocktopk_decode_step",
    "(Tensor q, Tensor k, Tensor v, Tensor(a!) kv_cache, Tensor(b!) kbar, Tensor page_indices, Tensor page_indptr, "
    "Tensor last_page_len, int topk, Tensor(c!)? sel_pages, Tensor(d!)? sel_count, float sm_scale, "
    "int sink_pages=0, int local_tokens=1, int first_page_offset=0, Tensor(e!)? workspace=None, "
    "Tensor? slot_ids=None) -> Tensor",
)


@torch.library.impl("kinetics::blocktopk_decode_step", "cuda")
def _step_impl(q, k, v, kv_cache, kbar, page_indices, page_indptr, last_page_len, topk, sel_pages, sel_count, sm_scale,
               sink_pages=0, local_tokens=1, first_page_offset=0, workspace=None, slot_ids=None):
    return blocktopk_decode_step(q, k, v, kv_cache, kbar, page_indices, page_indptr, last_page_len, topk,
                                 sel_pages=sel_pages, sel_count=sel_count, sm_scale=sm_scale, sink_pages=sink_pages,
                                 local_tokens=local_tokens, first_page_offset=first_page_offset, workspace=workspace,
                                 slot_ids=slot_ids)


@torch.library.register_fake("kinetics::blocktopk_decode_step")
def _step_fake(q, k, v, kv_cache, kbar, page_indices, page_indptr, last_page_len, topk, sel_pages, sel_count, sm_scale,
               sink_pages=0, local_tokens=1, first_page_offset=0, workspace=None, slot_ids=None):
    return torch.empty_like(q)


@torch.library.impl("kinetics::append_paged_kv", "cuda")
def _append_impl(k, v, kv_cache, kbar, page_indices, page_indptr, last_page_len, slot_ids=None):
    append_paged_kv(k, v, kv_cache, kbar, page_indices, page_indptr, last_page_len, slot_ids=slot_ids)


@torch.library.register_fake("kinetics::append_paged_kv")
def _append_fake(k, v, kv_cache, kbar, page_indices, page_indptr, last_page_len, slot_ids=None):
    return None


@torch.library.impl("kinetics::update_kv", "cuda")
def _update_kv_impl(k, v, kv_append_indptr, kv_cache, kv_page_indices, kv_page_indptr, cachelen, kbar=None, slot_ids=None):
    append_paged_kv_ragged(k, v, kv_append_indptr, kv_cache, kbar, kv_page_indices, kv_page_indptr, cachelen, slot_ids=slot_ids)


@torch.library.register_fake("kinetics::update_kv")
def _update_kv_fake(k, v, kv_append_indptr, kv_cache, kv_page_indices, kv_page_indptr, cachelen, kbar=None, slot_ids=None):
    return None


@torch.library.impl("kinetics::block_score_topk", "cuda")
def _select_impl(q, kbar, page_indices, page_indptr, last_page_len, topk, sel_pages, sel_count, sink_pages=0,
                 local_tokens=1, workspace=None, page_size=PAGE_SIZE, slot_ids=None):
    block_score_topk(q, kbar, page_indices, page_indptr, last_page_len, topk, sel_pages, sel_count,
                     sink_pages=sink_pages, local_tokens=local_tokens, workspace=workspace, page_size=page_size,
                     slot_ids=slot_ids)


@torch.library.register_fake("kinetics::block_score_topk")
def _select_fake(q, kbar, page_indices, page_indptr, last_page_len, topk, sel_pages, sel_count, sink_pages=0,
                 local_tokens=1, workspace=None, page_size=PAGE_SIZE, slot_ids=None):
    return None


@torch.library.impl("kinetics::sparse_paged_decode", "cuda")
def _sparse_impl(q, kv_cache, sel_pages, sel_count, last_page_len, workspace, sm_scale, num_splits, first_page_offset=0):
    return sparse_paged_decode(q, kv_cache, sel_pages, sel_count, last_page_len, workspace=workspace,
                               sm_scale=sm_scale, num_splits=num_splits, first_page_offset=first_page_offset)


@torch.library.register_fake("kinetics::sparse_paged_decode")
def _sparse_fake(q, kv_cache, sel_pages, sel_count, last_page_len, workspace, sm_scale, num_splits, first_page_offset=0):
    return torch.empty_like(q)


@torch.library.impl("kinetics::dense_paged_decode", "cuda")
def _dense_impl(q, kv_cache, page_indices, page_indptr, last_page_len, max_pages_per_seq, workspace, sm_scale, num_splits,
                first_page_offset=0):
    return dense_paged_decode(q, kv_cache, page_indices, page_indptr, last_page_len, max_pages_per_seq,
                              workspace=workspace, sm_scale=sm_scale, num_splits=num_splits,
                              first_page_offset=first_page_offset)


@torch.library.register_fake("kinetics::dense_paged_decode")
def _dense_fake(q, kv_cache, page_indices, page_indptr, last_page_len, max_pages_per_seq, workspace, sm_scale, num_splits,
                first_page_offset=0):
    return torch.empty_like(q)


# The reference's norm ops with their names and argument order
# (mylib::layer_norm, mylib::qk_norm, mylib::fused_layer_norm;
# benchmark/model_utils.py:4-41), plus the two fused row-wise steps.
torch.library.define("kinetics::layer_norm", "(Tensor hidden_states, float eps, Tensor weight) -> Tensor")
torch.library.define("kinetics::qk_norm", "(Tensor hidden_states, float eps, Tensor weight) -> Tensor")
torch.library.define("kinetics::fused_layer_norm",
                     "(Tensor hidden_states, Tensor(a!) residual, float eps, Tensor weight) -> Tensor")
torch.library.define("kinetics::qkv_norm_split",
                     "(Tensor qkv, Tensor q_weight, Tensor k_weight, float eps, int num_q_heads, int num_kv_heads) "
                     "-> (Tensor, Tensor, Tensor)")
torch.library.define("kinetics::gated_act", "(Tensor gate, Tensor up, str act) -> Tensor")


@torch.library.impl("kinetics::layer_norm", "cuda")
def _layer_norm_impl(hidden_states, eps, weight):
    return rms_norm(hidden_states, weight, eps)


@torch.library.register_fake("kinetics::layer_norm")
def _layer_norm_fake(hidden_states, eps, weight):
    return torch.empty_like(hidden_states)


@torch.library.impl("kinetics::qk_norm", "cuda")
def _qk_norm_impl(hidden_states, eps, weight):
    return rms_norm(hidden_states, weight, eps)


@torch.library.register_fake("kinetics::qk_norm")
def _qk_norm_fake(hidden_states, eps, weight):
    return torch.empty_like(hidden_states)


@torch.library.impl("kinetics::fused_layer_norm", "cuda")
def _fused_layer_norm_impl(hidden_states, residual, eps, weight):
    return rms_norm(hidden_states, weight, eps, residual=residual)


@torch.library.register_fake("kinetics::fused_layer_norm")
def _fused_layer_norm_fake(hidden_states, residual, eps, weight):
    return torch.empty_like(hidden_states)


@torch.library.impl("kinetics::qkv_norm_split", "cuda")
def _qkv_norm_split_impl(qkv, q_weight, k_weight, eps, num_q_heads, num_kv_heads):
    return qkv_norm_split(qkv, q_weight, k_weight, eps, num_q_heads, num_kv_heads)


@torch.library.register_fake("kinetics::qkv_norm_split")
def _qkv_norm_split_fake(qkv, q_weight, k_weight, eps, num_q_heads, num_kv_heads):
    batch = qkv.numel() // qkv.shape[-1]
    head_dim = q_weight.numel()
    return (qkv.new_empty(batch, num_q_heads, head_dim), qkv.new_empty(batch, num_kv_heads, head_dim),
            qkv.new_empty(batch, num_kv_heads, head_dim))


@torch.library.impl("kinetics::gated_act", "cuda")
def _gated_act_impl(gate, up, act):
    return gated_act(gate, up, act)


@torch.library.register_fake("kinetics::gated_act")
def _gated_act_fake(gate, up, act):
    return torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
