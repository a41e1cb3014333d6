"""The LiteSys-style KV manager (kinetics_amd/batch_cache.py) against the
oracle and against a contiguous-cache restatement of LiteSys' flow
(LiteSys/litesys/attention/batch_cache.py:86-168)."""
import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import blocktopk_oracle as O
from tests import problems as P

pytestmark = pytest.mark.gpu
DEV = "cuda"
D, PS = P.HEAD_DIM, P.PAGE_SIZE


_DT = [torch.bfloat16]   # element type of the test that is running (test_prefill_then_decode_like_litesys switches it)


def bf(x):
    return x.to(_DT[0])


class use_head_dim:
    """``with use_head_dim(64): ...`` -- the helpers of this module build configurations and tensors
    with head rows of that many elements (LiteSys reads head_dim from the model config,
    LiteSys/litesys/attention/batch_cache.py:27)."""

    def __init__(self, d):
        self.d = d

    def __enter__(self):
        global D
        self.prev, D = D, self.d

    def __exit__(self, *exc):
        global D
        D = self.prev
        return False


def cfg_small():
    return SimpleNamespace(num_attention_heads=4, num_key_value_heads=2, head_dim=D, hidden_size=512, num_hidden_layers=2)


def make_manager(**sparse):
    from kinetics_amd.batch_cache import PagedBatchKVManager

    block_policy = "attn_block_topk" in sparse and "attn_stride" not in sparse
    page = sparse.get("attn_block_size", PS) if block_policy else PS
    return PagedBatchKVManager(cfg_small(), max_batch_size=6, max_seq_len=page * 24, device=DEV, dtype=_DT[0], **sparse)


def test_rejects_what_it_does_not_implement():
    from kinetics_amd.batch_cache import PagedBatchKVManager

    cfg = SimpleNamespace(num_attention_heads=4, num_key_value_heads=2, head_dim=D, hidden_size=512, num_hidden_layers=1)
    with pytest.raises(NotImplementedError):
        PagedBatchKVManager(cfg, 2, 64, DEV, torch.bfloat16, attn_random_select=8, attn_local=4)
    with pytest.raises(NotImplementedError):
        PagedBatchKVManager(cfg, 2, 64, DEV, torch.bfloat16, attn_stride=8, attn_local=4)
    with pytest.raises(AssertionError):
        PagedBatchKVManager(cfg, 2, 64, DEV, torch.bfloat16, attn_topk=8, attn_block_topk=2, attn_local=4)
    with pytest.raises(AssertionError):
        PagedBatchKVManager(cfg, 2, 64, DEV, torch.bfloat16, attn_block_topk=2)          # LiteSys: local required
    with pytest.raises(NotImplementedError):
        PagedBatchKVManager(cfg, 2, 64, DEV, torch.bfloat16, attn_block_topk=2, attn_local=4, attn_block_size=24)
    # head rows of 64 elements: every policy; other sizes: nothing
    cfg64 = SimpleNamespace(num_attention_heads=4, num_key_value_heads=2, head_dim=64, hidden_size=256, num_hidden_layers=1)
    for policy in (dict(attn_block_topk=2, attn_local=4), dict(attn_topk=8, attn_local=4), dict(attn_local=4),
                   dict(attn_block_topk=2, attn_local=4, attn_stride=8)):
        PagedBatchKVManager(cfg64, 2, 64, DEV, torch.bfloat16, **policy)
    cfg96 = SimpleNamespace(num_attention_heads=4, num_key_value_heads=2, head_dim=96, hidden_size=384, num_hidden_layers=1)
    with pytest.raises(NotImplementedError, match="head_dim 96"):
        PagedBatchKVManager(cfg96, 2, 64, DEV, torch.bfloat16)


_POLICIES = [(dict(), None), (dict(attn_block_topk=3, attn_local=16), True),
             (dict(attn_block_topk=3, attn_local=16), False),
             (dict(attn_block_topk=2, attn_local=21), True),
             (dict(attn_block_topk=2, attn_local=20, attn_block_size=32), True),
             (dict(attn_block_topk=2, attn_local=33, attn_block_size=32), False),
             (dict(attn_block_topk=1, attn_local=7, attn_block_size=64), True),
             (dict(attn_block_topk=1, attn_local=40, attn_block_size=128), True),
             (dict(attn_block_topk=2, attn_local=9, attn_block_size=128), False),
             (dict(attn_local=24), False),
             (dict(attn_topk=40, attn_local=10), None),
             (dict(attn_block_topk=2, attn_local=9, attn_stride=8), None),
             (dict(attn_block_topk=3, attn_local=5, attn_stride=4, attn_block_size=8), None)]


_CASES = [(s, f, hd) for hd in (128, 64) for s, f in _POLICIES]


@pytest.mark.parametrize("sparse,fused,head_dim", _CASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_prefill_then_decode_like_litesys(sparse, fused, dtype, head_dim):
    _DT[0] = dtype
    try:
        with O.element_format("f16" if dtype is torch.float16 else "bf16"), use_head_dim(head_dim):   # how the oracle reads the cache bits
            _prefill_then_decode_like_litesys(sparse, fused)
    finally:
        _DT[0] = torch.bfloat16


def _prefill_then_decode_like_litesys(sparse, fused):
    torch.manual_seed(5)
    m = make_manager(**sparse)
    PS = m.page                   # tokens per page: LiteSys' block size for the block policy, else 16
    m._force_fused = fused        # both routes of decode(): one launch, or append + select + attend (None: the manager's choice)
    L, Hq, Hkv = 2, 4, 2
    hist = {}  # (layer, slot) -> (K [t, Hkv, D], V) float32 of the bf16 values fed so far

    strided = "attn_stride" in sparse
    window_only = bool(sparse) and "attn_block_topk" not in sparse and "attn_topk" not in sparse
    token_policy = "attn_topk" in sparse or strided or window_only
    policy = "strided" if strided else ("topk" if token_policy else "block")
    block_size, stride = sparse.get("attn_block_size", 16), sparse.get("attn_stride", 8)
    pad = PS - 4 if sparse and not token_policy else 0
    topk_block, local = sparse.get("attn_block_topk", sparse.get("attn_topk", 0)), sparse.get("attn_local")
    gen = torch.Generator().manual_seed(11)
    block_bias = torch.randn(64, Hkv, 1, generator=gen) * 0.5   # separates the block scores well beyond bf16 rounding

    def keys(slot_len, n, bsz=1):
        """n new key rows per sequence that start at token slot_len: N(0,1) plus
        a per-(LiteSys block, head) shift."""
        t = torch.arange(slot_len, slot_len + n)
        blk = torch.clamp((t - 4) // PS + 1, min=0)
        return bf(torch.randn(bsz, Hkv, n, D) + block_bias[blk].permute(1, 0, 2)[None]).to(DEV)

    def feed(layer, slot, k, v):  # k, v: [Hkv, s, D] bf16
        K, V = hist.get((layer, slot), (torch.zeros(0, Hkv, D), torch.zeros(0, Hkv, D)))
        hist[(layer, slot)] = (torch.cat([K, k.float().cpu().transpose(0, 1)]), torch.cat([V, v.float().cpu().transpose(0, 1)]))

    def dense_ref(layer, slot, q):  # q [Hq, s, D]; causal over history
        K, V = hist[(layer, slot)]
        s, total = q.shape[1], K.shape[0]
        out = torch.zeros(Hq, s, D)
        for hq in range(Hq):
            h = hq // 2
            logits = q[hq].float().cpu() @ K[:, h].T / math.sqrt(D)
            pos = torch.arange(total - s, total)[:, None]
            logits = logits.masked_fill(torch.arange(total)[None, :] > pos, float("-inf"))
            out[hq] = torch.softmax(logits, -1) @ V[:, h]
        return out

    # ---- prefill three requests, one at a time, in two chunks for slot 5 (append to history)
    for slot, lens in ((0, [PS * 7 + 5]), (2, [PS * 3]), (5, [PS * 2 + 1, PS * 6 + 9])):
        for s in lens:
            for layer in range(L):
                q, v = bf(torch.randn(1, Hq, s, D, device=DEV)), bf(torch.randn(1, Hkv, s, D, device=DEV))
                k = keys(int(m.kv_offset[layer][slot].item()), s)
                feed(layer, slot, k[0], v[0])
                out = m.compute_attention(q, k, v, layer, torch.tensor([slot]))
                assert out.shape == (1, s, Hq * D)
                want = dense_ref(layer, slot, q[0]).transpose(0, 1).reshape(1, s, Hq * D)
                assert torch.allclose(out.float().cpu(), want, rtol=2e-2, atol=2e-2)
    assert m.kv_offset[0].cpu().tolist() == [PS * 7 + 5, 0, PS * 3, 0, 0, PS * 8 + 10]

    def decode_round(batch_slots):
        for layer in range(L):
            bsz = len(batch_slots)
            q, v = bf(torch.randn(bsz, Hq, 1, D, device=DEV)), bf(torch.randn(bsz, Hkv, 1, D, device=DEV))
            k = torch.cat([keys(int(m.kv_offset[layer][slot].item()), 1) for slot in batch_slots])
            kv_before, kbar_before = P.from_torch(m.kv_cache[layer]), P.from_torch(m.kbar[layer])
            off_before = m.kv_offset[layer].cpu().numpy().copy()
            out = m.compute_attention(q, k, v, layer, torch.tensor(batch_slots))
            torch.cuda.synchronize()
            assert out.shape == (bsz, 1, Hq * D)
            for i, slot in enumerate(batch_slots):
                feed(layer, slot, k[i], v[i])
            # the paged cache holds exactly the history that was fed (pages through the slot's page list)
            table = m.pool.slot_table.cpu().numpy()
            owned = m.pool.slot_npages.cpu().numpy()
            for slot in batch_slots:
                K, V = hist[(layer, slot)]
                t = K.shape[0]
                assert m.kv_offset[layer][slot].item() == t == off_before[slot] + 1
                assert owned[slot] == (t + pad + PS - 1) // PS
                pages = torch.from_numpy(table[slot, : owned[slot]]).long().to(DEV)
                got_k = m.kv_cache[layer][pages, 0].reshape(-1, Hkv, D)[pad:pad + t].float().cpu()
                assert torch.equal(got_k, K)
            # oracle on the manager's own state before the call: the page table lists the ACTIVE
            # sequences in batch order, the mean keys stay with their slots
            lens = (off_before[batch_slots] + 1 + pad).astype(np.int64)
            n_pages = (lens + PS - 1) // PS
            indptr = np.zeros(bsz + 1, dtype=np.int32)
            indptr[1:] = np.cumsum(n_pages)
            idx = np.concatenate([table[s, : n_pages[i]] for i, s in enumerate(batch_slots)]).astype(np.int32)
            last = (lens - (n_pages - 1) * PS).astype(np.int32)
            assert np.array_equal(m._indptr.cpu().numpy()[: bsz + 1], indptr)
            assert np.array_equal(m.page_indices.cpu().numpy()[: len(idx)], idx)
            assert np.array_equal(m._last.cpu().numpy()[:bsz], last)
            qf, kf, vf = P.from_torch(q[:, :, 0]), P.from_torch(k[:, :, 0]), P.from_torch(v[:, :, 0])
            kbar_slots_before = kbar_before
            kbar_before = np.ascontiguousarray(kbar_slots_before[batch_slots])   # the oracle indexes mean keys by sequence
            is_sparse = bool(sparse) and layer not in (0,)   # layer 0 stays dense (attn_layer_skip default)
            if is_sparse and token_policy:
                O.append_paged_kv(kf, vf, kv_before, None, idx, indptr, last)
                want, keeps, _ = O.token_topk_decode(qf, kv_before, idx, indptr, last, topk_block, sink=4, local=local,
                                                     policy=policy, block_size=block_size, stride=stride)
                assert strided or not keeps[0].all() or lens[0] <= 4 + topk_block + local
            elif is_sparse:
                # the paged oracle on the manager's own state: one sink page, `local` newest tokens, 12 padding slots
                res = O.decode_step(qf, kf, vf, kv_before, kbar_before, idx, indptr, last, topk_block,
                                    sink_pages=1, local_tokens=local, first_page_offset=pad)
                want = res["out"]
                # really sparse for the long sequences: fewer pages than the context has
                assert res["sel_count"].max() < n_pages.max()
            else:
                O.append_paged_kv(kf, vf, kv_before, kbar_before, idx, indptr, last)
                want, _ = O.dense_paged_decode(qf, kv_before, idx, indptr, last, first_page_offset=pad)
            assert np.array_equal(P.from_torch(m.kv_cache[layer]), kv_before)
            if not token_policy:   # (that policy has no use for mean keys and does not maintain them)
                want_kbar = kbar_slots_before.copy()
                want_kbar[batch_slots] = kbar_before        # the active slots' rows, and nobody else's
                assert np.array_equal(P.from_torch(m.kbar[layer]), want_kbar)
            got = out.float().cpu().numpy().reshape(bsz, Hq, D)
            err = np.abs(got - want)
            assert np.all(err <= 2e-2 + 2e-2 * np.abs(want))
            # and LiteSys' own formulation on the contiguous history that was fed: full logits, its mask
            # (4 sink tokens, blocks from token 4, `local` newest tokens), softmax, P.V
            for i, slot in enumerate(batch_slots):
                K, V = hist[(layer, slot)]
                ref, keep = O.litesys_decode(q[i, :, 0].float().cpu().numpy(), K.numpy(), V.numpy(),
                                             topk_block if is_sparse else None, local, policy=policy,
                                             block_size=block_size, stride=stride)
                if is_sparse and K.shape[0] > 100 * max(block_size, 16) // 16:
                    assert not keep.all()
                assert np.all(np.abs(got[i] - ref) <= 2e-2 + 2e-2 * np.abs(ref)), (layer, slot)

    for _ in range(12):           # crosses page boundaries (mean keys refreshed) for every slot
        decode_round([0, 2, 5])
    decode_round([5, 0])          # a subset, in another order
    free_before, _ = m.pool.status()
    held = int(m.pool.slot_npages[2].item())
    m.clear_cache(2)              # recycle slot 2: its pages go back to the pool
    assert m.kv_offset[1][2].item() == 0
    assert m.pool.status() == (free_before + held, 0) and int(m.pool.slot_npages[2].item()) == 0
    for layer in range(L):
        hist.pop((layer, 2))
        q, k, v = bf(torch.randn(1, Hq, 20, D, device=DEV)), bf(torch.randn(1, Hkv, 20, D, device=DEV)), bf(torch.randn(1, Hkv, 20, D, device=DEV))
        feed(layer, 2, k[0], v[0])
        m.compute_attention(q, k, v, layer, torch.tensor([2]))
    decode_round([2, 5])


@pytest.mark.parametrize("batch,with_slots", [(0, False), (1, False), (7, True), (1500, True), (3000, False)])
def test_slot_page_table_against_numpy(batch, with_slots):
    """CSR page table of a slot-based cache (kin_build_slot_page_table): empty
    sequences, sequences longer than a slot's run (they get an empty list: nothing
    may be appended into a cut one), more sequences than one scan pass, an empty batch."""
    from kinetics_amd import ops

    rng = np.random.default_rng(batch + 1)
    pps = 24
    lens = rng.integers(-3, PS * pps + 40, size=batch).astype(np.int32)
    if batch >= 7:
        lens[:4] = [0, 1, PS * pps, PS * pps + 17]
    slots = rng.permutation(batch + 5)[:batch].astype(np.int32) if with_slots else None
    idx = torch.full((max(batch * pps, 1),), -1, dtype=torch.int32, device=DEV)
    ptr = torch.full((batch + 1,), -1, dtype=torch.int32, device=DEV)
    last = torch.full((batch,), -1, dtype=torch.int32, device=DEV)
    ops.build_slot_page_table(torch.from_numpy(lens).to(DEV), pps, PS, idx, ptr, last,
                              slot_ids=None if slots is None else torch.from_numpy(slots).to(DEV))
    torch.cuda.synchronize()
    n = (np.maximum(lens, 0) + PS - 1) // PS
    n = np.where(n > pps, 0, n)
    want_ptr = np.concatenate([[0], np.cumsum(n)]).astype(np.int32)
    assert np.array_equal(ptr.cpu().numpy(), want_ptr)
    want_last = np.where(n > 0, np.maximum(lens, 0) - (n - 1) * PS, 1).astype(np.int32)
    assert np.array_equal(last.cpu().numpy(), want_last)
    got = idx.cpu().numpy()
    for b in range(batch):
        s = b if slots is None else int(slots[b])
        assert np.array_equal(got[want_ptr[b]: want_ptr[b + 1]], s * pps + np.arange(n[b]))


def test_page_pool_against_a_python_free_list():
    """kin_page_pool_init / reserve / release / kin_build_pool_page_table against a
    Python model of the same free list on a random sequence of grow, release and
    over-subscription steps: page lists, counts, free stack and status word."""
    from kinetics_amd import ops

    rng = np.random.default_rng(77)
    slots, pps, pool_pages = 37, 9, 120
    pool = ops.PagePool(pool_pages, slots, pps, PS, DEV)
    stack = list(range(pool_pages - 1, -1, -1))
    table = [[] for _ in range(slots)]
    status = 0
    idx = torch.empty(pool_pages, dtype=torch.int32, device=DEV)
    ptr = torch.empty(slots + 1, dtype=torch.int32, device=DEV)
    last = torch.empty(slots, dtype=torch.int32, device=DEV)
    for step in range(60):
        if step % 5 == 4:
            rel = rng.permutation(slots)[: int(rng.integers(1, 6))].astype(np.int32)
            pool.release(torch.from_numpy(rel).to(DEV))
            for s in rel:
                stack.extend(table[s])
                table[s] = []
        lens = np.where(rng.random(slots) < 0.4, rng.integers(0, PS * pps + 30, size=slots), 0).astype(np.int32)
        if step == 20:
            lens[:] = PS * pps       # more than the pool holds: nothing may be reserved
        pool.reserve(torch.from_numpy(lens).to(DEV))
        need = np.minimum((lens + PS - 1) // PS, pps)
        extra = [max(0, int(need[s]) - len(table[s])) for s in range(slots)]
        if (lens > PS * pps).any():
            status |= 2
        if sum(extra) > len(stack):
            status |= 1
        else:
            top, first = len(stack), 0
            for s in range(slots):
                table[s] += [stack[top - 1 - (first + j)] for j in range(extra[s])]
                first += extra[s]
            del stack[top - first:]
        free, bits = pool.status()
        assert (free, bits) == (len(stack), status), f"step {step}"
        assert pool.slot_npages.cpu().tolist() == [len(t) for t in table], f"step {step}"
        got_table = pool.slot_table.cpu().numpy()
        for s in range(slots):
            assert got_table[s, : len(table[s])].tolist() == table[s], f"step {step} slot {s}"
        assert sorted(pool.free_stack.cpu().numpy()[:free].tolist() + [p for t in table for p in t]) == list(range(pool_pages))
        # the CSR table of these lengths: a sequence its slot cannot hold (a failed reserve, or longer
        # than a slot may grow) has an empty list
        pool.build_page_table(torch.from_numpy(lens).to(DEV), idx, ptr, last)
        full = (np.maximum(lens, 0) + PS - 1) // PS
        n = np.array([int(full[s]) if int(full[s]) <= len(table[s]) else 0 for s in range(slots)])
        want_ptr = np.concatenate([[0], np.cumsum(n)])
        assert ptr.cpu().tolist() == want_ptr.tolist()
        got = idx.cpu().numpy()
        for s in range(slots):
            assert got[want_ptr[s]: want_ptr[s + 1]].tolist() == table[s][: n[s]]
    assert status == 3     # both conditions were met on the way
    with pytest.raises(Exception):
        pool.raise_on_overflow()
    pool.raise_on_overflow()   # reported once: the bits were cleared
    assert pool.status()[1] == 0


def test_page_pool_skips_bad_and_repeated_slot_ids():
    """Slot ids outside the pool, or named twice in one call, are skipped and flagged; the
    free list stays whole (free pages + owned pages = every page, once)."""
    from kinetics_amd import ops

    slots, pps, pool_pages = 8, 6, 40
    pool = ops.PagePool(pool_pages, slots, pps, PS, DEV)

    def whole():
        free, _ = pool.status()
        owned = pool.slot_npages.cpu().tolist()
        table = pool.slot_table.cpu().numpy()
        pages = pool.free_stack.cpu().numpy()[:free].tolist() + [int(p) for s in range(slots) for p in table[s, : owned[s]]]
        return sorted(pages) == list(range(pool_pages)), owned

    ids = torch.tensor([3, 9, 3, -1, 5, 3], dtype=torch.int32, device=DEV)       # 9 and -1 do not exist, 3 comes three times
    lens = torch.tensor([PS * 2, PS, PS * 2, PS, PS * 3 + 1, PS * 2], dtype=torch.int32, device=DEV)
    pool.reserve(lens, ids)
    ok, owned = whole()
    assert ok and owned == [0, 0, 0, 2, 0, 4, 0, 0]                              # one entry of slot 3 counts, not three
    assert pool.status()[1] == ops.PagePool.BAD_SLOT
    idx = torch.full((pool_pages,), -1, dtype=torch.int32, device=DEV)
    ptr = torch.empty(7, dtype=torch.int32, device=DEV)
    last = torch.empty(6, dtype=torch.int32, device=DEV)
    pool.build_page_table(lens, idx, ptr, last, ids)
    # sequences with an unusable id have an empty list (the table itself does not look for repeats)
    assert ptr.cpu().tolist() == [0, 2, 2, 4, 4, 8, 10]
    with pytest.raises(ValueError):
        pool.raise_on_overflow()
    pool.release(torch.tensor([3, 3, 11, 5], dtype=torch.int32, device=DEV))    # a repeat and a stranger
    ok, owned = whole()
    assert ok and owned == [0] * 8 and pool.status() == (pool_pages, ops.PagePool.BAD_SLOT)


def test_manager_with_a_small_pool_and_overlong_sequences():
    """A pool smaller than max_batch x max_len serves what fits, reuses returned pages
    (the recycled slot's table is fragmented) and reports exhaustion and sequences
    past max_seq_len instead of silently overwriting the last slot."""
    from kinetics_amd._lib import KineticsError

    torch.manual_seed(9)
    L, Hq, Hkv = 2, 4, 2
    from kinetics_amd.batch_cache import PagedBatchKVManager

    m = PagedBatchKVManager(cfg_small(), max_batch_size=4, max_seq_len=PS * 6, device=DEV, dtype=torch.bfloat16,
                            kv_pool_pages=10)
    assert m.kv_cache[0].shape[0] == 10

    def prefill(slot, n):
        for layer in range(L):
            q, k, v = (bf(torch.randn(1, h, n, D, device=DEV)) for h in (Hq, Hkv, Hkv))
            m.compute_attention(q, k, v, layer, torch.tensor([slot]))

    prefill(0, PS * 4)            # 4 pages
    prefill(1, PS * 3 + 1)        # 4 pages
    assert m.pool.status() == (2, 0)
    with pytest.raises(KineticsError):
        prefill(2, PS * 3)        # wants 3, 2 are free
    # the failed request left nothing behind: no pages, no offset, no status bit to trip over later
    assert m.pool.status() == (2, 0) and m.kv_offset[0][2].item() == 0 and int(m.pool.slot_npages[2].item()) == 0
    m.clear_cache(0)              # 4 pages back
    assert m.pool.status() == (6, 0)
    prefill(2, PS * 5)            # takes 5 of the 6 free pages, most of them slot 0's old ones
    pages2 = m.pool.slot_table[2, :5].cpu().tolist()
    assert sorted(pages2) != pages2 or pages2[0] != 0   # not the fixed run a slot used to own
    # decode slot 1 until it is past max_seq_len: flagged, and from then on inert -- its pages and mean
    # keys are never written again (it used to be cut to the pages it owned, and every further token
    # overwrote the last slot of its last page)
    m.clear_cache(2)
    snap, outs = None, []
    for step in range(PS * 3 + 4):
        if int(m.kv_offset[0][1].item()) == PS * 6:        # the slot is full: what it holds now must stay
            pages1 = m.pool.slot_table[1, : int(m.pool.slot_npages[1].item())].long()
            snap = [(c[pages1].clone(), kb[1].clone()) for c, kb in zip(m.kv_cache, m.kbar)]
        for layer in range(L):
            q, k, v = (bf(torch.randn(1, h, 1, D, device=DEV)) for h in (Hq, Hkv, Hkv))
            out = m.compute_attention(q, k, v, layer, torch.tensor([1]))
            if snap is not None:
                outs.append(out)
    assert m.kv_offset[0][1].item() > PS * 6 and snap is not None and len(outs) >= 8
    for layer in range(L):
        assert torch.equal(m.kv_cache[layer][pages1], snap[layer][0]) and torch.equal(m.kbar[layer][1], snap[layer][1])
    assert all(bool((o == 0).all()) for o in outs)         # an empty page list attends nothing
    with pytest.raises(ValueError):
        m.clear_cache(1)
    assert m.pool.status()[1] == 0
    m.clear_cache(1)                                       # reported once; the slot is usable again
    prefill(1, PS * 2)
    assert m.pool.status()[1] == 0 and int(m.pool.slot_npages[1].item()) == 2


@pytest.mark.parametrize("sparse", [dict(), dict(attn_block_topk=2, attn_local=18), dict(attn_block_topk=2, attn_local=18, attn_block_size=32)])
def test_float16_manager(sparse):
    """LiteSys' manager takes a dtype (batch_cache.py:21); in float16 the paged manager
    must give LiteSys' own formulation (full logits, its mask, softmax, P.V) on the
    history that was fed."""
    from kinetics_amd.batch_cache import PagedBatchKVManager

    torch.manual_seed(21)
    L, Hq, Hkv = 2, 4, 2
    block = sparse.get("attn_block_size", 16)
    m = PagedBatchKVManager(cfg_small(), max_batch_size=3, max_seq_len=block * 30, device=DEV, dtype=torch.float16, **sparse)
    hist = {}
    gen = torch.Generator().manual_seed(3)
    bias = torch.randn(64, Hkv, 1, generator=gen) * 0.5

    def keys(start, n):
        t = torch.arange(start, start + n)
        blk = torch.clamp((t - 4) // block + 1, min=0)
        return (torch.randn(1, Hkv, n, D) + bias[blk].permute(1, 0, 2)[None]).half().to(DEV)

    def feed(layer, slot, k, v):
        K, V = hist.get((layer, slot), (torch.zeros(0, Hkv, D), torch.zeros(0, Hkv, D)))
        hist[(layer, slot)] = (torch.cat([K, k.float().cpu().transpose(0, 1)]), torch.cat([V, v.float().cpu().transpose(0, 1)]))

    for slot, n in ((0, block * 9 + 3), (2, block * 5)):
        for layer in range(L):
            q, v = torch.randn(1, Hq, n, D, device=DEV).half(), torch.randn(1, Hkv, n, D, device=DEV).half()
            k = keys(0, n)
            feed(layer, slot, k[0], v[0])
            out = m.compute_attention(q, k, v, layer, torch.tensor([slot]))
            assert out.dtype is torch.float16 and out.shape == (1, n, Hq * D)
    for _ in range(block + 2):                     # crosses a page boundary: a float16 mean key is written
        for layer in range(L):
            slots = [0, 2]
            q, v = torch.randn(2, Hq, 1, D, device=DEV).half(), torch.randn(2, Hkv, 1, D, device=DEV).half()
            k = torch.cat([keys(int(m.kv_offset[layer][s].item()), 1) for s in slots])
            out = m.compute_attention(q, k, v, layer, torch.tensor(slots))
            torch.cuda.synchronize()
            got = out.float().cpu().numpy().reshape(2, Hq, D)
            for i, s in enumerate(slots):
                feed(layer, s, k[i], v[i])
                K, V = hist[(layer, s)]
                is_sparse = bool(sparse) and layer != 0
                ref, keep = O.litesys_decode(q[i, :, 0].float().cpu().numpy(), K.numpy(), V.numpy(),
                                             sparse["attn_block_topk"] if is_sparse else None, sparse.get("attn_local"),
                                             block_size=block)
                assert np.all(np.abs(got[i] - ref) <= 2e-2 + 2e-2 * np.abs(ref)), (layer, s)
                if is_sparse:
                    assert not keep.all()


def _fed_manager(max_batch, sparse, seed, prefill_lens):
    """A manager after seeded prefills; returns it with the fp32 history per (layer, slot)."""
    from kinetics_amd.batch_cache import PagedBatchKVManager

    L, Hq, Hkv = 2, 4, 2
    m = PagedBatchKVManager(cfg_small(), max_batch_size=max_batch, max_seq_len=PS * 24, device=DEV, dtype=torch.bfloat16, **sparse)
    gen = torch.Generator().manual_seed(seed)
    hist = {}
    for slot, n in prefill_lens:
        for layer in range(L):
            q, k, v = (torch.randn(1, h, n, D, generator=gen).bfloat16().to(DEV) for h in (Hq, Hkv, Hkv))
            hist[(layer, slot)] = (k[0].float().cpu().transpose(0, 1), v[0].float().cpu().transpose(0, 1))
            m.compute_attention(q, k, v, layer, torch.tensor([slot]))
    return m, hist


@pytest.mark.parametrize("head_dim", [128, 64])
@pytest.mark.parametrize("sparse", [dict(), dict(attn_block_topk=3, attn_local=16)])
def test_manager_few_active_slots_in_any_order(sparse, head_dim):
    with use_head_dim(head_dim):
        _manager_few_active_slots_in_any_order(sparse)


def _manager_few_active_slots_in_any_order(sparse):
    """Five active slots of a 40-slot manager, in an order that is not the slots': q, k, v and the
    output follow the batch, the caches the slots.  The page table built by the first layer of a
    step is reused by the second (same batch_idx object) -- same bits as rebuilding it -- and the
    outputs are LiteSys' own formulation on the fed history."""
    L, Hq, Hkv = 2, 4, 2
    slots = [33, 4, 17, 29, 8]
    pre = [(s, PS * (3 + i) + 2 * i + 1) for i, s in enumerate(slots)]
    a, hist = _fed_manager(40, sparse, 31, pre)
    b, _ = _fed_manager(40, sparse, 31, pre)
    gen = torch.Generator().manual_seed(32)
    same = torch.tensor(slots)
    for step in range(PS + 3):                                   # every slot crosses a page boundary
        order = slots if step % 2 == 0 else slots[::-1][:3]      # a subset in another order now and then
        batch_a = same if order is slots else torch.tensor(order)
        for layer in range(L):
            q, k, v = (torch.randn(len(order), h, 1, D, generator=gen).bfloat16().to(DEV) for h in (Hq, Hkv, Hkv))
            out_a = a.compute_attention(q, k, v, layer, batch_a)                 # one object for the whole step
            out_b = b.compute_attention(q, k, v, layer, torch.tensor(order))     # a new one per layer: rebuilt each time
            torch.cuda.synchronize()
            assert torch.equal(out_a, out_b), (step, layer)
            got = out_a.float().cpu().numpy().reshape(len(order), Hq, D)
            for i, s in enumerate(order):
                K, V = hist[(layer, s)]
                K, V = torch.cat([K, k[i].float().cpu().transpose(0, 1)]), torch.cat([V, v[i].float().cpu().transpose(0, 1)])
                hist[(layer, s)] = (K, V)
                is_sparse = bool(sparse) and layer != 0
                ref, _ = O.litesys_decode(q[i, :, 0].float().cpu().numpy(), K.numpy(), V.numpy(),
                                          sparse["attn_block_topk"] if is_sparse else None, sparse.get("attn_local"))
                assert np.all(np.abs(got[i] - ref) <= 2e-2 + 2e-2 * np.abs(ref)), (step, layer, s)
    for layer in range(L):
        assert torch.equal(a.kv_cache[layer], b.kv_cache[layer]) and torch.equal(a.kbar[layer], b.kbar[layer])
        assert torch.equal(a.kv_offset[layer], b.kv_offset[layer])
    assert a.pool.status() == b.pool.status() and a.pool.status()[1] == 0


def test_manager_decode_step_replays_under_hip_graph():
    """A whole decode step of the manager (every layer: offsets, page reservation, page table, the
    attention kernels) recorded once as a HIP graph: every replay, with the program's own eager work
    and synchronisations in between, equals an eager twin fed the same inputs."""
    L, Hq, Hkv = 2, 4, 2
    sparse = dict(attn_block_topk=3, attn_local=16)
    slots = [6, 1, 9]
    pre = [(6, PS * 5 + 3), (1, PS * 8), (9, PS * 3 + 15)]
    g, _ = _fed_manager(12, sparse, 41, pre)
    e, _ = _fed_manager(12, sparse, 41, pre)
    batch_idx = torch.tensor(slots, device=DEV)
    qs = [torch.zeros(3, Hq, 1, D, dtype=torch.bfloat16, device=DEV) for _ in range(L)]
    ks = [torch.zeros(3, Hkv, 1, D, dtype=torch.bfloat16, device=DEV) for _ in range(L)]
    vs = [torch.zeros(3, Hkv, 1, D, dtype=torch.bfloat16, device=DEV) for _ in range(L)]

    def step(m):
        return [m.compute_attention(qs[layer], ks[layer], vs[layer], layer, batch_idx) for layer in range(L)]

    gen = torch.Generator(device=DEV).manual_seed(42)

    def new_inputs():
        for t in qs + ks + vs:
            t.copy_(torch.randn(t.shape, generator=gen, device=DEV).bfloat16())

    new_inputs()
    step(g), step(e)                                  # warm-up on both (one token each)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    new_inputs()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            outs_g = step(g)                          # (capture runs nothing: the first replay is this step)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for trial in range(PS + 2):                       # page boundaries are crossed inside replays
        if trial:
            new_inputs()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs_g]
        want = step(e)
        torch.cuda.synchronize()
        for layer in range(L):
            assert torch.equal(got[layer], want[layer]), f"replay {trial}, layer {layer}"
    for layer in range(L):
        assert torch.equal(g.kv_offset[layer], e.kv_offset[layer])
        assert torch.equal(g.kbar[layer], e.kbar[layer])
    assert g.pool.status() == e.pool.status() and g.pool.slot_npages.tolist() == e.pool.slot_npages.tolist()
