"""Pins the CPU oracle (oracle/blocktopk_oracle.py, oracle/torch_path.py).

The reference ships no tests, golden vectors or fixtures for this path, so the
oracle is pinned by library routines (torch bf16 casts, torch.topk, torch SDPA,
scipy logsumexp) and by what the mathematics fixes (closed forms, invariants,
brute force on small inputs).  Every check is chosen so that a plausible slip
-- wrong slot, transposed operand, dropped scale, off-by-one page, wrong mask --
breaks it.  No GPU needed.
"""
import math

import numpy as np
import pytest
import torch
from scipy.special import logsumexp

from oracle import blocktopk_oracle as O
from oracle import torch_path
from tests import problems as P

D, PS = P.HEAD_DIM, P.PAGE_SIZE


# --------------------------------------------------------------------------- bf16


def test_bf16_roundtrip_matches_torch():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(4096).astype(np.float32) * 10,
        np.array([0.0, -0.0, 1.0, -1.0, 65504.0, 1e-40, 3.3895314e38, np.inf, -np.inf], dtype=np.float32),
        # exact ties between two bf16 values: must round to even
        np.array([1.00390625, 1.01171875, -1.00390625], dtype=np.float32),
    ])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = O.f32_to_bf16(x)
    assert np.array_equal(got, want)
    back = torch.from_numpy(got.view(np.int16)).view(torch.bfloat16).float().numpy()
    assert np.array_equal(O.bf16_to_f32(got), back)
    nan = O.f32_to_bf16(np.array([np.nan], dtype=np.float32))
    assert np.isnan(O.bf16_to_f32(nan))[0]


# --------------------------------------------------------------------------- append


@pytest.mark.parametrize("residue", list(range(PS)))
def test_append_writes_exactly_one_slot(residue):
    # one length per residue class of L mod page_size, random page table
    lengths = [3 * PS + residue + 1, residue + 1, 7 * PS + residue + 1]
    pb = P.make_problem(100 + residue, lengths, num_kv_heads=2, group=2)
    before = pb.kv_cache.copy()
    kbar = pb.kbar.copy()
    O.append_paged_kv(pb.k, pb.v, pb.kv_cache, kbar, pb.page_indices, pb.page_indptr, pb.last_page_len)
    changed = np.zeros(pb.kv_cache.shape[:3], dtype=bool)
    for b, L in enumerate(lengths):
        pages = O.seq_pages(pb.page_indices, pb.page_indptr, b)
        pid, pos = pages[(L - 1) // PS], (L - 1) % PS  # closed form of "last token's slot"
        assert np.array_equal(pb.kv_cache[pid, 0, pos], pb.k[b])
        assert np.array_equal(pb.kv_cache[pid, 1, pos], pb.v[b])
        changed[pid, :, pos] = True
    # every other byte is untouched
    assert np.array_equal(pb.kv_cache[~changed], before[~changed])
    # kbar changes only where a page became full
    for b, L in enumerate(lengths):
        n_pages = (L + PS - 1) // PS
        if L % PS == 0:
            pages = O.seq_pages(pb.page_indices, pb.page_indptr, b)
            want = O.page_mean_key(pb.kv_cache[pages[-1], 0].transpose(1, 0, 2))
            assert np.array_equal(kbar[b, :, n_pages - 1], want)
            mask = np.ones(kbar.shape[2], dtype=bool)
            mask[n_pages - 1] = False
            assert np.array_equal(kbar[b][:, mask], pb.kbar[b][:, mask])
        else:
            assert np.array_equal(kbar[b], pb.kbar[b])


def test_append_skips_empty_sequences():
    pb = P.make_problem(7, [0, 5, 0, 33])
    before = pb.kv_cache.copy()
    O.append_paged_kv(pb.k, pb.v, pb.kv_cache, None, pb.page_indices, pb.page_indptr, pb.last_page_len)
    assert (pb.kv_cache != before).any(axis=(1, 2, 3, 4)).sum() == 2  # exactly two pages touched


def test_page_mean_key_against_float64_and_closed_forms():
    rng = np.random.default_rng(3)
    pages = P.randn_bf16(rng, (64, PS, D), scale=3.0)
    got = O.bf16_to_f32(O.page_mean_key(pages)).astype(np.float64)
    exact = O.bf16_to_f32(pages).astype(np.float64).mean(axis=1)
    ulp = np.maximum(np.abs(exact), 2.0 ** -126) * 2.0 ** -7  # one bf16 ulp is <= 2^-7 relative
    assert np.all(np.abs(got - exact) <= ulp)
    # constant rows: the mean is that row, exactly
    row = P.randn_bf16(rng, (1, D))
    assert np.array_equal(O.page_mean_key(np.repeat(row, PS, axis=0)), row[0])
    # a single non-zero row of value 16*x gives x
    z = np.zeros((PS, D), dtype=np.uint16)
    z[5] = O.f32_to_bf16(np.full(D, 48.0, dtype=np.float32))
    assert np.array_equal(O.bf16_to_f32(O.page_mean_key(z)), np.full(D, 3.0, dtype=np.float32))


def test_build_kbar_covers_full_pages_only():
    pb = P.make_problem(11, [PS * 4, PS * 2 + 3, 1, 0], num_kv_heads=2, group=1, build_kbar=False)
    sentinel = np.uint16(0x7FC0)
    kbar = np.full_like(pb.kbar, sentinel)
    O.build_kbar(pb.kv_cache, kbar, pb.page_indices, pb.page_indptr, pb.last_page_len)
    full = [4, 2, 0, 0]
    for b in range(4):
        pages = O.seq_pages(pb.page_indices, pb.page_indptr, b)
        for p in range(kbar.shape[2]):
            if p < full[b]:
                for h in range(2):
                    want = O.page_mean_key(pb.kv_cache[pages[p], 0, :, h, :])
                    assert np.array_equal(kbar[b, h, p], want)
            else:
                assert np.all(kbar[b, :, p] == sentinel)


def _ragged_case(seed, before, new, hkv=2, slack=2):
    """A cache holding ``before[b]`` tokens per sequence, the table after
    appending ``new[b]`` more, and the rows to append."""
    rng = np.random.default_rng(seed)
    after = [a + n for a, n in zip(before, new)]
    pb = P.make_problem(seed, after, num_kv_heads=hkv, group=1, kbar_slack=slack)
    nnz = sum(new)
    k, v = P.randn_bf16(rng, (nnz, hkv, D)), P.randn_bf16(rng, (nnz, hkv, D))
    append_indptr = np.concatenate([[0], np.cumsum(new)]).astype(np.int32)
    return pb, k, v, append_indptr, after


def test_ragged_append_equals_token_by_token_append():
    """The multi-token append is the single-token append (pinned above) applied
    once per new token with the table of that moment; nothing else changes."""
    before = [0, 5, PS * 2, PS * 3 + 15, 40, 7, PS]
    new = [PS * 2 + 3, 1, 0, 18, PS * 4, 9, PS]
    pb, k, v, append_indptr, after = _ragged_case(77, before, new)
    kv_a, kbar_a = pb.kv_cache.copy(), pb.kbar.copy()
    O.append_paged_kv_ragged(k, v, append_indptr, kv_a, kbar_a, pb.page_indices, pb.page_indptr, pb.last_page_len)
    kv_b, kbar_b = pb.kv_cache.copy(), pb.kbar.copy()
    for b in range(pb.B):
        pages = O.seq_pages(pb.page_indices, pb.page_indptr, b)
        for i in range(new[b]):
            length = before[b] + i + 1
            n_pages = (length + PS - 1) // PS
            one_k = np.zeros((1, pb.Hkv, D), dtype=np.uint16)
            one_v = np.zeros_like(one_k)
            one_k[0], one_v[0] = k[append_indptr[b] + i], v[append_indptr[b] + i]
            sub_kbar = kbar_b[b : b + 1]
            O.append_paged_kv(one_k, one_v, kv_b, sub_kbar, pages[:n_pages].astype(np.int32),
                              np.array([0, n_pages], dtype=np.int32), np.array([length - (n_pages - 1) * PS], dtype=np.int32))
    assert np.array_equal(kv_a, kv_b)
    assert np.array_equal(kbar_a, kbar_b)
    # rows land where the closed form says, bit for bit
    for b in range(pb.B):
        pages = O.seq_pages(pb.page_indices, pb.page_indptr, b)
        for i in range(new[b]):
            pos = before[b] + i
            assert np.array_equal(kv_a[pages[pos // PS], 0, pos % PS], k[append_indptr[b] + i])
            assert np.array_equal(kv_a[pages[pos // PS], 1, pos % PS], v[append_indptr[b] + i])
    # bytes outside the appended rows are untouched
    touched = np.zeros(kv_a.shape[:3], dtype=bool)
    for b in range(pb.B):
        pages = O.seq_pages(pb.page_indices, pb.page_indptr, b)
        for i in range(new[b]):
            pos = before[b] + i
            touched[pages[pos // PS], :, pos % PS] = True
    assert np.array_equal(kv_a[~touched], pb.kv_cache[~touched])


# --------------------------------------------------------------------------- scores


def test_scores_identities():
    pb = P.make_problem(21, [PS * 9 + 4, PS * 5 + 1], num_kv_heads=2, group=4)
    sc = O.block_scores(pb.q, pb.kbar, pb.page_indptr, pb.last_page_len)
    qf = O.bf16_to_f32(pb.q).astype(np.float64)
    for b in range(pb.B):
        n_cand = (pb.lengths[b] + PS - 1) // PS - 1
        for h in range(2):
            assert sc[b][h].shape == (n_cand,)
            # mean_g (q_g . k) == (mean_g q_g) . k
            qbar = qf[b, 4 * h : 4 * h + 4].mean(axis=0)
            kb = O.bf16_to_f32(pb.kbar[b, h, :n_cand]).astype(np.float64)
            assert np.allclose(sc[b][h], kb @ qbar, rtol=1e-12, atol=1e-12)
            # not the other head's keys, not the other head's queries
            other = O.bf16_to_f32(pb.kbar[b, 1 - h, :n_cand]).astype(np.float64) @ qbar
            assert not np.allclose(sc[b][h], other)


def test_scores_equal_litesys_group_mean_then_block_mean():
    """LiteSys ranks blocks by mean over the query group, then mean over the
    block's tokens, of q.k/sqrt(D) (sparsity_utils.py:36-37).  With keys whose
    page mean is exactly representable this equals score/sqrt(D)."""
    rng = np.random.default_rng(5)
    n_pages, G = 6, 4
    # small integers: sums and the /16 mean are exact in bf16
    K = (rng.integers(-8, 9, size=(n_pages, PS, D)) * 16).astype(np.float32)
    kv = np.zeros((n_pages + 1, 2, PS, 1, D), dtype=np.uint16)
    kv[:n_pages, 0, :, 0] = O.f32_to_bf16(K)
    indices = np.arange(n_pages + 1, dtype=np.int32)
    indptr = np.array([0, n_pages + 1], dtype=np.int32)
    kbar = np.zeros((1, 1, n_pages + 1, D), dtype=np.uint16)
    O.build_kbar(kv, kbar, indices, indptr, np.array([1], dtype=np.int32))
    q = P.randn_bf16(rng, (1, G, D))
    sc = O.block_scores(q, kbar, indptr, np.array([1], dtype=np.int32))[0][0]
    logits = np.einsum("gd,ptd->gpt", O.bf16_to_f32(q[0]).astype(np.float64), K.astype(np.float64)) / math.sqrt(D)
    litesys = logits.mean(axis=0).mean(axis=-1)
    assert np.allclose(sc / math.sqrt(D), litesys, rtol=1e-12, atol=1e-12)


# --------------------------------------------------------------------------- selection


def test_select_topk_against_library_routines():
    rng = np.random.default_rng(9)
    for n, k in [(1, 1), (5, 3), (257, 64), (2048, 128), (100, 100), (100, 250)]:
        s = rng.standard_normal(n)
        got = O.select_topk(s, k)
        kk = min(k, n)
        want_t = torch.topk(torch.from_numpy(s), kk).indices.numpy()
        assert np.array_equal(got, want_t)  # distinct values: order is fixed too
        part = np.argpartition(-s, kk - 1)[:kk]
        assert set(got.tolist()) == set(part.tolist())


def test_select_topk_tie_break_is_lowest_index():
    assert O.select_topk(np.zeros(10), 4).tolist() == [0, 1, 2, 3]
    s = np.array([1.0, 5.0, 5.0, 2.0, 5.0, 0.0])
    assert O.select_topk(s, 2).tolist() == [1, 2]
    assert O.select_topk(s, 4).tolist() == [1, 2, 4, 3]
    assert O.select_topk(np.array([]), 3).tolist() == []


def test_block_score_topk_page_list_layout():
    pb = P.make_problem(31, [PS * 20 + 7, PS * 3, 1, 0, PS * 2 + 1], topk=4)
    sel, cnt, logical, scores = O.block_score_topk(pb.q, pb.kbar, pb.page_indices, pb.page_indptr, pb.last_page_len, pb.topk)
    assert sel.shape == (5, 1, 5)
    assert cnt[:, 0].tolist() == [5, 3, 1, 0, 3]  # min(k, n_cand) + 1, 0 for the empty sequence
    for b in range(5):
        pages = O.seq_pages(pb.page_indices, pb.page_indptr, b)
        c = cnt[b, 0]
        if c == 0:
            assert np.all(sel[b] == -1)
            continue
        assert sel[b, 0, c - 1] == pages[-1]                # last page always attended, applied once
        assert np.array_equal(sel[b, 0, : c - 1], pages[logical[b][0]])  # logical -> physical, once
        assert np.all(sel[b, 0, c:] == -1)
        assert pages[-1] not in sel[b, 0, : c - 1]          # the last page is not a candidate
        s = scores[b][0]
        if len(s) > c - 1:
            assert s[logical[b][0]].min() >= np.delete(s, logical[b][0]).max()


def test_selection_matches_rule():
    s = np.array([10.0, 9.0, 5.0, 5.0 + 1e-6, 1.0])
    assert O.selection_matches([0, 1, 3], s, 3)[0]
    assert O.selection_matches([0, 1, 2], s, 3)[0]        # tie within 1e-3 relative
    assert not O.selection_matches([0, 1, 4], s, 3)[0]    # 1.0 is no tie of 5.0
    assert not O.selection_matches([0, 1], s, 3)[0]
    assert not O.selection_matches([0, 0, 1], s, 3)[0]
    assert not O.selection_matches([0, 1, 7], s, 3)[0]


# --------------------------------------------------------------------------- attention


def _depaged(pb, b, h):
    pages = O.seq_pages(pb.page_indices, pb.page_indptr, b)
    L = int(pb.lengths[b])
    d = pb.kv_cache.shape[4]
    K = O.elem_to_f32(pb.kv_cache[pages, 0, :, h]).reshape(-1, d)[:L]
    V = O.elem_to_f32(pb.kv_cache[pages, 1, :, h]).reshape(-1, d)[:L]
    return K.astype(np.float64), V.astype(np.float64)


def test_float16_element_format_is_ieee_half():
    """The oracle's float16 conversions against torch's: bit patterns and values."""
    x = np.random.default_rng(5).standard_normal(4096).astype(np.float32) * np.float32(300.0)
    x[:4] = [0.0, -0.0, 65504.0, 1e-7]
    with O.element_format("f16"):
        bits = O.f32_to_elem(x)
        back = O.elem_to_f32(bits)
        mean = O.page_mean_key(bits.reshape(-1, 16, 16))          # [256 pages, 16 rows, 16 cols]
    t = torch.from_numpy(x).half()
    assert np.array_equal(bits, t.view(torch.int16).numpy().view(np.uint16))
    assert np.array_equal(back, t.float().numpy())
    want = (t.float().reshape(-1, 16, 16).sum(dim=1) * (1.0 / 16)).half()   # fp32 sum of 16 rows (exact order aside), one rounding
    got = torch.from_numpy(mean.view(np.int16)).view(torch.float16)
    assert torch.allclose(got.float(), want.float(), rtol=2 ** -10, atol=1e-6)
    assert O._ELEMENT_FORMAT == "bf16"                            # the block restored the default


@pytest.mark.parametrize("head_dim", [128, 64])
@pytest.mark.parametrize("fmt", ["bf16", "f16"])
@pytest.mark.parametrize("page_size", [16, 32, 64, 128])
def test_dense_attention_equals_torch_sdpa(page_size, fmt, head_dim):
    """Head rows of 64 elements too (LiteSys reads head_dim from the model config,
    LiteSys/litesys/attention/batch_cache.py:27): the scale follows the row length."""
    with O.element_format(fmt), P.head_dim(head_dim):
        _dense_attention_equals_torch_sdpa(page_size, head_dim)


def _dense_attention_equals_torch_sdpa(page_size, D=D):
    pb = P.make_problem(41, [PS * 6 + 5, PS * 2, 9], num_kv_heads=2, group=4, page_size=page_size)
    assert pb.kv_cache.shape[2] == page_size and pb.kv_cache.shape[4] == D and pb.q.shape[2] == D
    out, lse = O.dense_paged_decode(pb.q, pb.kv_cache, pb.page_indices, pb.page_indptr, pb.last_page_len)
    qf = O.elem_to_f32(pb.q).astype(np.float64)
    for b in range(pb.B):
        for h in range(2):
            K, V = _depaged(pb, b, h)
            qt = torch.from_numpy(qf[b, 4 * h : 4 * h + 4])[None, :, None, :]       # [1, G, 1, D]
            Kt = torch.from_numpy(K)[None, None].expand(1, 4, -1, -1)
            Vt = torch.from_numpy(V)[None, None].expand(1, 4, -1, -1)
            want = torch.nn.functional.scaled_dot_product_attention(qt, Kt, Vt)[0, :, 0].numpy()
            assert np.allclose(out[b, 4 * h : 4 * h + 4], want, rtol=1e-9, atol=1e-9)
            logits = qf[b, 4 * h : 4 * h + 4] @ K.T / math.sqrt(D)
            assert np.allclose(lse[b, 4 * h : 4 * h + 4], logsumexp(logits, axis=1), rtol=1e-12)


def test_repaging_leaves_dense_attention_unchanged():
    """The same token rows stored in 16-, 32- and 64-token pages: dense attention
    over them is the same function of the tokens, bit for bit in float64 up to
    summation order."""
    rng = np.random.default_rng(47)
    lengths = [257, 64, 5]
    Hkv, G = 2, 3
    rows_k = [P.randn_bf16(rng, (L, Hkv, D)) for L in lengths]
    rows_v = [P.randn_bf16(rng, (L, Hkv, D)) for L in lengths]
    q = P.randn_bf16(rng, (len(lengths), Hkv * G, D))
    outs = []
    for ps in (16, 32, 64, 128):
        n_pages = [(L + ps - 1) // ps for L in lengths]
        total = sum(n_pages) + 2
        perm = rng.permutation(total).astype(np.int32)
        kv = P.randn_bf16(rng, (total, 2, ps, Hkv, D))
        indptr = np.concatenate([[0], np.cumsum(n_pages)]).astype(np.int32)
        for b, L in enumerate(lengths):
            for t in range(L):
                pid = perm[indptr[b] + t // ps]
                kv[pid, 0, t % ps], kv[pid, 1, t % ps] = rows_k[b][t], rows_v[b][t]
        last = np.array([L - (n - 1) * ps for L, n in zip(lengths, n_pages)], dtype=np.int32)
        outs.append(O.dense_paged_decode(q, kv, perm[: indptr[-1]], indptr, last))
    for o, l in outs[1:]:
        assert np.allclose(o, outs[0][0], rtol=1e-12, atol=1e-14) and np.allclose(l, outs[0][1], rtol=1e-12)


def test_sparse_with_every_page_selected_equals_dense():
    pb = P.make_problem(43, [PS * 5 + 2, PS * 3 + 16], num_kv_heads=1, group=4, topk=64)
    sel, cnt, _, _ = O.block_score_topk(pb.q, pb.kbar, pb.page_indices, pb.page_indptr, pb.last_page_len, pb.topk)
    a, la = O.sparse_paged_decode(pb.q, pb.kv_cache, sel, cnt, pb.last_page_len)
    d, ld = O.dense_paged_decode(pb.q, pb.kv_cache, pb.page_indices, pb.page_indptr, pb.last_page_len)
    assert np.allclose(a, d, rtol=1e-10, atol=1e-12) and np.allclose(la, ld, rtol=1e-12)


def test_attention_closed_forms():
    rng = np.random.default_rng(47)
    pb = P.make_problem(47, [1, PS * 4 + 3], num_kv_heads=1, group=4, topk=2)
    O.append_paged_kv(pb.k, pb.v, pb.kv_cache, pb.kbar, pb.page_indices, pb.page_indptr, pb.last_page_len)
    sel, cnt, _, _ = O.block_score_topk(pb.q, pb.kbar, pb.page_indices, pb.page_indptr, pb.last_page_len, pb.topk)
    out, lse = O.sparse_paged_decode(pb.q, pb.kv_cache, sel, cnt, pb.last_page_len)
    # one token: softmax over one logit is 1 -> out is that token's value, lse its logit
    v0 = O.bf16_to_f32(pb.v[0, 0]).astype(np.float64)
    assert np.allclose(out[0], np.broadcast_to(v0, (4, D)), rtol=0, atol=1e-12)
    logit = O.bf16_to_f32(pb.q[0]).astype(np.float64) @ O.bf16_to_f32(pb.k[0, 0]).astype(np.float64) / math.sqrt(D)
    assert np.allclose(lse[0], logit, rtol=1e-12)
    # constant V: out is that constant whatever the weights
    cv = P.randn_bf16(rng, (D,))
    kv2 = pb.kv_cache.copy()
    kv2[:, 1] = cv
    out2, _ = O.sparse_paged_decode(pb.q, kv2, sel, cnt, pb.last_page_len)
    assert np.allclose(out2, O.bf16_to_f32(cv).astype(np.float64), rtol=0, atol=1e-12)
    # q = 0: uniform weights -> mean of the attended values (2 full pages + 3 tokens of the last)
    q0 = np.zeros_like(pb.q)
    out3, lse3 = O.sparse_paged_decode(q0, pb.kv_cache, sel, cnt, pb.last_page_len)
    pages = sel[1, 0, : cnt[1, 0]]
    V = O.bf16_to_f32(pb.kv_cache[pages, 1, :, 0]).reshape(-1, D)[: 2 * PS + 3].astype(np.float64)
    assert np.allclose(out3[1], V.mean(axis=0), rtol=1e-12, atol=1e-12)
    assert np.allclose(lse3[1], math.log(2 * PS + 3), rtol=1e-12)


def test_attention_permutation_and_split_invariance():
    pb = P.make_problem(53, [PS * 12 + 9], num_kv_heads=1, group=4, topk=7)
    sel, cnt, _, _ = O.block_score_topk(pb.q, pb.kbar, pb.page_indices, pb.page_indptr, pb.last_page_len, pb.topk)
    out, lse = O.sparse_paged_decode(pb.q, pb.kv_cache, sel, cnt, pb.last_page_len)
    # shuffle the full pages (the final, partial page keeps its place)
    c = cnt[0, 0]
    sel2 = sel.copy()
    sel2[0, 0, : c - 1] = sel[0, 0, : c - 1][::-1]
    out2, lse2 = O.sparse_paged_decode(pb.q, pb.kv_cache, sel2, cnt, pb.last_page_len)
    assert np.allclose(out, out2, rtol=1e-12, atol=1e-13) and np.allclose(lse, lse2, rtol=1e-13)
    # any partition of the page list merged by (out, lse) gives the same answer
    qf = O.bf16_to_f32(pb.q[0]).astype(np.float64)
    pages = sel[0, 0, :c]
    for cuts in ([3], [1, 2, 5], [c - 1]):
        outs, lses = [], []
        bounds = [0, *cuts, c]
        for lo, hi in zip(bounds[:-1], bounds[1:]):
            ll = pb.last_page_len[0] if hi == c else PS
            o, l = O.attend_pages(qf, pb.kv_cache, pages[lo:hi], 0, ll, 1 / math.sqrt(D))
            outs.append(o)
            lses.append(l)
        # an empty part must be neutral
        outs.append(np.zeros_like(outs[0]))
        lses.append(np.full_like(lses[0], -np.inf))
        mo, ml = O.merge_partials(outs, lses)
        assert np.allclose(mo, out[0], rtol=1e-12, atol=1e-13) and np.allclose(ml, lse[0], rtol=1e-13)


def test_decode_step_equals_masked_dense_formulation_float16():
    with O.element_format("f16"):
        test_decode_step_equals_masked_dense_formulation(32)


def test_decode_step_equals_masked_dense_formulation_head_dim_64():
    with P.head_dim(64):
        test_decode_step_equals_masked_dense_formulation(16, D=64)
        test_decode_step_equals_masked_dense_formulation(64, D=64)


@pytest.mark.parametrize("page_size", [16, 32, 64, 128])
def test_decode_step_equals_masked_dense_formulation(page_size, D=D):
    """LiteSys expresses block sparsity as a -inf mask on full-context logits
    (sparsity_utils.py:39-45) followed by softmax and P.V; the gather form must
    give the same numbers, at every page size (the reference's --page_size,
    benchmark/blocktopk.py:13)."""
    PS = page_size
    pb = P.make_problem(59, [PS * 10 + 5, PS * 7 + PS], num_kv_heads=2, group=2, topk=3, page_size=page_size)
    res = O.decode_step(pb.q, pb.k, pb.v, pb.kv_cache, pb.kbar, pb.page_indices, pb.page_indptr, pb.last_page_len, pb.topk)
    qf = O.elem_to_f32(pb.q).astype(np.float64)
    for b in range(pb.B):
        L = int(pb.lengths[b])
        n_pages = (L + PS - 1) // PS
        for h in range(2):
            K, V = _depaged(pb, b, h)
            keep = np.zeros(n_pages * PS, dtype=bool)
            for p in res["sel_logical"][b][h]:
                keep[p * PS : (p + 1) * PS] = True
            keep[(n_pages - 1) * PS :] = True
            keep = keep[:L]
            logits = qf[b, 2 * h : 2 * h + 2] @ K.T / math.sqrt(D)
            logits[:, ~keep] = -np.inf
            w = np.exp(logits - logits.max(axis=1, keepdims=True))
            w /= w.sum(axis=1, keepdims=True)
            assert np.allclose(res["out"][b, 2 * h : 2 * h + 2], w @ V, rtol=1e-10, atol=1e-12)


# --------------------------------------------------------------------------- torch path


def test_torch_path_agrees_with_oracle():
    B, n_pages, topk = 4, 40, 8
    pb = P.make_problem(61, [PS * (n_pages - 1) + 6] * B, num_kv_heads=1, group=4, topk=topk)
    kv_t = P.to_torch(pb.kv_cache.copy())
    table = torch.from_numpy(pb.page_indices.astype(np.int64)).reshape(B, n_pages)
    out_t, idx_t = torch_path.blocktopk_decode_step(
        P.to_torch(pb.q), P.to_torch(pb.k), P.to_torch(pb.v), kv_t, P.to_torch(pb.kbar[:, 0, : n_pages - 1]),
        table, torch.from_numpy(pb.last_page_len.astype(np.int64)), topk)
    res = O.decode_step(pb.q, pb.k, pb.v, pb.kv_cache, pb.kbar, pb.page_indices, pb.page_indptr, pb.last_page_len, topk)
    assert np.array_equal(P.from_torch(kv_t), pb.kv_cache)  # same append
    for b in range(B):
        ok, msg = O.selection_matches(idx_t[b].numpy(), res["scores"][b][0], topk)
        assert ok, msg
    got = out_t.float().numpy().astype(np.float64)
    assert np.allclose(got, res["out"], rtol=2e-2, atol=2e-2)
    dense_t = torch_path.dense_decode_step(P.to_torch(pb.q), P.to_torch(pb.k), P.to_torch(pb.v), kv_t, table,
                                           torch.from_numpy(pb.last_page_len.astype(np.int64)))
    dense_o, _ = O.dense_paged_decode(pb.q, pb.kv_cache, pb.page_indices, pb.page_indptr, pb.last_page_len)
    assert np.allclose(dense_t.float().numpy(), dense_o, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("case", P.BF16_CASES, ids=lambda c: f"seed{c[0]}")
def test_selection_differs_from_the_references_bf16_scoring_only_by_its_rounding(case):
    """The reference ranks pages by bf16 scores (bf16 einsum output, bf16 mean:
    benchmark/blocktopk_decoder.py:216-217); this build ranks by fp32 / float64
    scores.  Where the two top-k sets differ, the reference's own scores of the
    swapped pages are tied within the reference's rounding band; sequences with the
    same page set give the same output within the 2e-2 contract."""
    seed, B, L, topk, G, sigma = case
    pb, n, table, last = P.bf16_case(*case)
    kv_t = P.to_torch(pb.kv_cache.copy())
    kbar_t = P.to_torch(pb.kbar[:, 0, :n])
    out_ref, idx_ref = torch_path.blocktopk_decode_step(P.to_torch(pb.q), P.to_torch(pb.k), P.to_torch(pb.v), kv_t, kbar_t, table,
                                                        last, topk, compute_dtype=torch.bfloat16)
    res = O.decode_step(pb.q, pb.k, pb.v, pb.kv_cache, pb.kbar, pb.page_indices, pb.page_indptr, pb.last_page_len, topk)
    got = torch.from_numpy(np.stack([res["sel_logical"][b][0] for b in range(B)]))
    cmp = torch_path.compare_with_bf16_reference(P.to_torch(pb.q), kbar_t, got, topk)
    assert torch.equal(cmp["ref_idx"].sort(dim=1).values, idx_ref.sort(dim=1).values)   # the helper ranks what the step ranks
    assert cmp["worst_violation"] <= 0.0, cmp
    assert cmp["overlap"] >= 0.98, cmp
    # Sequences whose page sets agree: the outputs agree within the contract.  A sequence where a
    # tied page was swapped attends other tokens, so its output moves by what those tokens weigh
    # (a property of top-k selection, not of the arithmetic): bounded loosely, and reported.
    same = (cmp["ref_idx"].sort(dim=1).values == got.sort(dim=1).values).all(dim=1).numpy()
    diff = np.abs(out_ref.float().numpy().astype(np.float64) - res["out"])
    tol = 2e-2 + 2e-2 * np.abs(res["out"])
    assert np.all(diff[same] <= tol[same]), f"same pages, output differs by {diff[same].max()}"
    if (~same).any():
        assert diff[~same].max() <= 0.1, f"swapped tie pages moved the output by {diff[~same].max()}"


def test_sink_and_local_pages_are_pinned_not_candidates():
    """Sink pages and the pages of the newest local tokens (LiteSys' sink and
    local window, sparsity_utils.py:24-35) are always in the list, never scored."""
    pb = P.make_problem(71, [PS * 20 + 7, PS * 4 + 2, PS * 2, 5, 0], topk=3)
    sel, cnt, logical, scores = O.block_score_topk(pb.q, pb.kbar, pb.page_indices, pb.page_indptr, pb.last_page_len, 3,
                                                   sink_pages=2, local_tokens=2 * PS + 1)
    assert sel.shape[2] == 3 + 2 + 3 == O.sel_list_capacity(3, 2, 2 * PS + 1)
    # n_pages = 21, 5, 2, 1, 0 -> (sink, cand, local) = (2,16,3), (2,0,3), (1,0,1), (0,0,1), -
    assert cnt[:, 0].tolist() == [3 + 5, 5, 2, 1, 0]
    pages = O.seq_pages(pb.page_indices, pb.page_indptr, 0)
    assert len(scores[0][0]) == 16
    assert sel[0, 0, :2].tolist() == [pages[0], pages[1]]                    # sink pages first
    assert sel[0, 0, 2:5].tolist() == pages[logical[0][0]].tolist()          # then the winners, best first
    assert sel[0, 0, 5:8].tolist() == [pages[18], pages[19], pages[20]]      # then the local pages, open page last
    assert all(2 <= i < 18 for i in logical[0][0])
    # scores are those of logical pages 2..17
    full = O.block_scores(pb.q, pb.kbar, pb.page_indptr, pb.last_page_len)[0][0]  # default split: candidates 0..19
    assert np.allclose(scores[0][0], full[2:18])
    # short sequences: everything pinned, in logical order, open page last
    p1 = O.seq_pages(pb.page_indices, pb.page_indptr, 1)
    assert sel[1, 0, :5].tolist() == p1.tolist()
    # attending to the pinned list equals the masked-dense formulation
    out, _ = O.sparse_paged_decode(pb.q, pb.kv_cache, sel, cnt, pb.last_page_len)
    K, V = _depaged(pb, 0, 0)
    keep = np.zeros(21 * PS, dtype=bool)
    for p_ in list(logical[0][0]) + [0, 1, 18, 19, 20]:
        keep[p_ * PS : (p_ + 1) * PS] = True
    keep = keep[: PS * 20 + 7]
    logits = O.bf16_to_f32(pb.q[0]).astype(np.float64) @ K.T / math.sqrt(D)
    logits[:, ~keep] = -np.inf
    w = np.exp(logits - logits.max(axis=1, keepdims=True))
    w /= w.sum(axis=1, keepdims=True)
    assert np.allclose(out[0], w @ V, rtol=1e-10, atol=1e-12)
    # defaults reproduce the reference rule
    a = O.block_score_topk(pb.q, pb.kbar, pb.page_indices, pb.page_indptr, pb.last_page_len, 3)
    b = O.block_score_topk(pb.q, pb.kbar, pb.page_indices, pb.page_indptr, pb.last_page_len, 3, sink_pages=0, local_tokens=1)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


@pytest.mark.parametrize("page_size", [16, 32, 64, 128])
def test_split_pages_against_token_level_definition(page_size):
    """Brute force: a page is a candidate iff it comes after the sink pages and
    ends at or before the first of the newest ``local_tokens`` tokens."""
    PS = page_size
    for kv_len in list(range(1, 300)) + [1000, 1009, 4096]:
        n_pages = (kv_len + PS - 1) // PS
        last = kv_len - (n_pages - 1) * PS
        for sink in (0, 1, 2, 5):
            for local in (1, 2, 15, 16, 17, 18, 33, 100):
                n_sink, n_cand, n_local = O.split_pages(n_pages, last, sink, local, 10 ** 6, PS)
                want_sink = min(sink, n_pages - 1)
                cand = [p for p in range(want_sink, n_pages) if (p + 1) * PS <= kv_len - local]
                assert (n_sink, n_cand) == (want_sink, len(cand)), (kv_len, sink, local)
                assert cand == list(range(want_sink, want_sink + len(cand)))
                assert n_sink + n_cand + n_local == n_pages and n_local >= 1
                assert n_local <= 1 + (local + PS - 2) // PS <= 1 + (local + 14) // 16
    # local_tokens = 16 (L - 1) + 1 pins exactly the last L pages whatever the open page holds
    for n_pages in range(1, 12):
        for last in range(1, PS + 1):
            for L in (1, 2, 3):
                n_sink, n_cand, n_local = O.split_pages(n_pages, last, 0, PS * (L - 1) + 1, 10 ** 6, PS)
                assert n_local == min(L, n_pages) and n_cand == n_pages - n_local
    # mean keys exist for the first kbar_pages pages only
    assert O.split_pages(100, 3, 2, 1, 50) == (2, 48, 1)


def test_litesys_mask_hand_case():
    """sparsity_utils.py:24-47 on a case small enough to do by hand: 57 tokens,
    sink 4, local 5, one block of 16 kept out of three."""
    seq_len, local = 4 + 3 * 16 + 5, 5
    mean_logits = np.zeros(seq_len)
    mean_logits[4 + 16 : 4 + 32] = 1.0      # block 1 has the largest mean
    mean_logits[4] = 10.0                    # one large token does not make block 0 win: mean 10/16 < 1
    keep = O.litesys_blockwise_topk_mask(mean_logits, seq_len, 1, local)
    want = np.zeros(seq_len, dtype=bool)
    want[:4] = True
    want[20:36] = True
    want[52:] = True
    assert np.array_equal(keep, want)
    # a non-aligned tail: the local part absorbs the remainder (58 tokens -> 6 local tokens)
    keep = O.litesys_blockwise_topk_mask(np.append(mean_logits, 0.0), seq_len + 1, 1, local)
    assert keep[52:].all() and keep[20:36].all() and keep.sum() == 4 + 16 + 6
    # at or below n_full = roundup16(4 + 5 + 16) = 32 tokens everything stays
    assert O.litesys_blockwise_topk_mask(np.zeros(32), 32, 1, local).all()
    assert O.litesys_blockwise_topk_mask(np.arange(33.0), 33, 1, local).sum() == 4 + 16 + 13


@pytest.mark.parametrize("page_size", [16, 32, 64, 128])
def test_page_lists_with_offset_12_equal_litesys_mask_formulation(page_size):
    """The paged formulation (sink_pages=1, local_tokens=local, sequences stored
    page_size - 4 slots into their first page: 12 for LiteSys' default blocks of 16) and
    LiteSys' mask on full logits with block_size = page_size
    (sparsity_utils.py:24-47, batch_cache.py:154-168) are the same function:
    same kept tokens, same output.  Keys are multiples of 64 so that page means
    are exact in bfloat16 and no score is perturbed by rounding."""
    rng = np.random.default_rng(123)
    PS = page_size
    Hkv, G, pad = 2, 2, page_size - 4
    for seq_len, topk, local in [(300, 3, 20), (301, 3, 16), (52, 2, 5), (53, 2, 5), (40, 4, 7), (5, 2, 3), (4, 1, 1),
                                 (1, 1, 1), (1000, 10, 64), (999, 10, 1), (131, 1, 100), (307, 5, 33)]:
        K = (rng.integers(-1, 2, size=(seq_len, Hkv, D)) * 64).astype(np.float32)
        V = O.bf16_to_f32(P.randn_bf16(rng, (seq_len, Hkv, D)))
        q = P.randn_bf16(rng, (1, Hkv * G, D))
        cache_len = seq_len + pad
        n_pages = (cache_len + PS - 1) // PS
        perm = rng.permutation(n_pages + 3).astype(np.int32)[:n_pages]
        kv = P.randn_bf16(rng, (n_pages + 3, 2, PS, Hkv, D))            # padding slots hold garbage
        flat_k = np.zeros((n_pages * PS, Hkv, D), dtype=np.uint16)
        flat_v = np.zeros_like(flat_k)
        flat_k[:pad], flat_v[:pad] = P.randn_bf16(rng, (pad, Hkv, D)), P.randn_bf16(rng, (pad, Hkv, D))
        flat_k[pad:cache_len], flat_v[pad:cache_len] = O.f32_to_bf16(K), O.f32_to_bf16(V)
        kv[perm, 0] = flat_k.reshape(n_pages, PS, Hkv, D)
        kv[perm, 1] = flat_v.reshape(n_pages, PS, Hkv, D)
        indptr = np.array([0, n_pages], dtype=np.int32)
        last = np.array([cache_len - (n_pages - 1) * PS], dtype=np.int32)
        kbar = np.zeros((1, Hkv, n_pages, D), dtype=np.uint16)
        O.build_kbar(kv, kbar, perm, indptr, last)
        sel, cnt, logical, _ = O.block_score_topk(q, kbar, perm, indptr, last, topk, sink_pages=1, local_tokens=local,
                                                  page_size=PS)
        out, _ = O.sparse_paged_decode(q, kv, sel, cnt, last, first_page_offset=pad)
        want, keep = O.litesys_decode(O.bf16_to_f32(q[0]), K, V, topk, local, block_size=PS)
        lookup = {int(p): i for i, p in enumerate(perm)}
        for h in range(Hkv):
            got_keep = np.zeros(n_pages * PS, dtype=bool)
            for pid in sel[0, h, : cnt[0, h]]:
                got_keep[lookup[int(pid)] * PS : (lookup[int(pid)] + 1) * PS] = True
            assert np.array_equal(got_keep[pad:cache_len], keep[h]), (seq_len, topk, local, h)
        assert np.allclose(out[0], want, rtol=1e-9, atol=1e-11), (seq_len, topk, local)
        # the dense layer (attn_layer_skip) on the same cache
        dense, _ = O.dense_paged_decode(q, kv, perm, indptr, last, first_page_offset=pad)
        want_dense, _ = O.litesys_decode(O.bf16_to_f32(q[0]), K, V, None, local)
        assert np.allclose(dense[0], want_dense, rtol=1e-9, atol=1e-11)


def test_litesys_token_topk_mask():
    """sparsity_utils.py:6-21 by hand and against torch.topk."""
    seq_len, local, sink, topk = 30, 3, 4, 5
    ml = np.zeros(seq_len)
    ml[[6, 9, 10, 20, 26]] = [5.0, 4.0, 3.0, 2.0, 1.0]
    ml[[1, 28]] = 100.0                      # sink / local tokens are not candidates
    keep = O.litesys_topk_mask(ml, seq_len, topk, local, sink)
    want = np.zeros(seq_len, dtype=bool)
    want[:4] = True
    want[27:] = True
    want[[6, 9, 10, 20, 26]] = True
    assert np.array_equal(keep, want)
    assert O.litesys_topk_mask(ml, 12, topk, local, sink).all()        # seq_len <= sink + topk + local: dense
    assert O.litesys_topk_mask(ml[:13], 13, topk, local, sink).sum() == 12
    rng = np.random.default_rng(3)
    for seq_len, topk, local in [(500, 64, 16), (77, 10, 1), (4096, 1024, 64)]:
        ml = rng.standard_normal(seq_len)
        keep = O.litesys_topk_mask(ml, seq_len, topk, local)
        idx = torch.topk(torch.from_numpy(ml[4 : seq_len - local]), topk).indices.numpy() + 4
        want = np.zeros(seq_len, dtype=bool)
        want[:4] = True
        want[seq_len - local :] = True
        want[idx] = True
        assert np.array_equal(keep, want)


def test_token_topk_decode_on_pages_is_litesys_on_the_contiguous_cache():
    """The paged wrapper only de-pages; with a budget that covers everything the
    result is dense attention; with first_page_offset the padding slots vanish."""
    pb = P.make_problem(88, [PS * 12 + 5, 9, PS * 3], num_kv_heads=2, group=2)
    O.append_paged_kv(pb.k, pb.v, pb.kv_cache, None, pb.page_indices, pb.page_indptr, pb.last_page_len)
    out, keeps, means = O.token_topk_decode(pb.q, pb.kv_cache, pb.page_indices, pb.page_indptr, pb.last_page_len, 10 ** 6)
    dense, _ = O.dense_paged_decode(pb.q, pb.kv_cache, pb.page_indices, pb.page_indptr, pb.last_page_len)
    assert np.allclose(out, dense, rtol=1e-10, atol=1e-12) and all(k.all() for k in keeps)
    out, keeps, means = O.token_topk_decode(pb.q, pb.kv_cache, pb.page_indices, pb.page_indptr, pb.last_page_len, 20,
                                            sink=4, local=8)
    assert keeps[0].sum(axis=1).tolist() == [32, 32] and keeps[1].all()
    K, V = _depaged(pb, 0, 1)
    q = O.bf16_to_f32(pb.q[0, 2:4]).astype(np.float64)
    logits = q @ K.T / math.sqrt(D)
    assert np.allclose(means[0][1], logits.mean(axis=0), rtol=1e-12)
    logits[:, ~keeps[0][1]] = -np.inf
    w = np.exp(logits - logits.max(axis=1, keepdims=True))
    assert np.allclose(out[0, 2:4], (w / w.sum(axis=1, keepdims=True)) @ V, rtol=1e-10, atol=1e-12)
    off, _, _ = O.token_topk_decode(pb.q, pb.kv_cache, pb.page_indices, pb.page_indptr, pb.last_page_len, 10 ** 6,
                                    first_page_offset=7)
    dense_off, _ = O.dense_paged_decode(pb.q, pb.kv_cache, pb.page_indices, pb.page_indptr, pb.last_page_len,
                                        first_page_offset=7)
    assert np.allclose(off, dense_off, rtol=1e-10, atol=1e-12)


def test_litesys_strided_mask():
    """sparsity_utils.py:49-105 by hand, including its quirks: twice the budget in
    blocks is chosen, the union is cut in POSITION order, and what no chosen block
    covers is dropped."""
    ml = np.zeros(17)
    ml[4:14] = [0, 0, 5, 5, 5, 5, 0, 0, 9, 9]          # the dynamic part (sink 4, local 3)
    ml[[0, 15]] = 50.0                                  # sink / local tokens are not candidates
    keep = O.litesys_strided_mask(ml, 17, 1, 3, sink=4, block_size=4, stride=2)
    # blocks [0,4) [2,6) [4,8) [6,10): means 2.5, 5, 2.5, 4.5 -> blocks 1 and 3 -> tokens 2..9 -> first 4: 2..5
    want = np.zeros(17, dtype=bool)
    want[:4] = True
    want[14:] = True
    want[4 + 2 : 4 + 6] = True
    assert np.array_equal(keep, want)
    assert np.allclose(O.strided_block_means(ml, 17, 3, sink=4, block_size=4, stride=2), [2.5, 5, 2.5, 4.5])
    # budget of two blocks: all four blocks are chosen, the first 8 united tokens stay, 8 and 9 are cut
    keep = O.litesys_strided_mask(ml, 17, 2, 3, sink=4, block_size=4, stride=2)
    assert keep[4:12].all() and not keep[12:14].any()
    # a tail no block reaches is dropped even with a huge budget: L = 11 -> still 4 blocks, token 10 uncovered
    keep = O.litesys_strided_mask(np.append(ml, 0.0), 18, 100, 3, sink=4, block_size=4, stride=2)
    assert keep[4:14].all() and not keep[14] and keep[15:].all()
    # too short for a block, or nothing dynamic: nothing masked
    assert O.litesys_strided_mask(ml, 10, 1, 3, sink=4, block_size=4, stride=2).all()
    assert O.litesys_strided_mask(ml, 7, 1, 3, sink=4, block_size=4, stride=2).all()
    # against a direct restatement with torch.topk on random data
    rng = np.random.default_rng(5)
    for seq_len, k, local, bs, st in [(500, 8, 16, 16, 8), (333, 5, 7, 16, 4), (2000, 30, 64, 16, 16), (90, 2, 1, 8, 3)]:
        ml = rng.standard_normal(seq_len)
        dyn = torch.from_numpy(ml[4 : seq_len - local])
        nb = (len(dyn) - bs) // st + 1
        means = dyn.unfold(0, bs, st).mean(dim=-1)
        assert means.shape[0] == nb
        top = torch.topk(means, min(2 * k, nb)).indices
        toks = torch.unique(torch.cat([torch.arange(i * st, i * st + bs) for i in top.tolist()]))[: k * bs]
        want = np.zeros(seq_len, dtype=bool)
        want[:4] = True
        want[seq_len - local :] = True
        want[4 + toks.numpy()] = True
        assert np.array_equal(O.litesys_strided_mask(ml, seq_len, k, local, 4, bs, st), want)


# --------------------------------------------------------------------------- layer row steps


def _ulps(a_bits, b_bits):
    """Largest distance between two bf16 arrays in units of the last place."""
    def key(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, 0x8000 - b, b)

    # values that differ by less than 1e-6 count as equal (fp32 against fp64 tails near zero)
    near = np.abs(O.bf16_to_f32(a_bits).astype(np.float64) - O.bf16_to_f32(b_bits)) <= 1e-6
    return int(np.where(near, 0, np.abs(key(a_bits) - key(b_bits))).max())


def test_rms_norm_against_torch_and_closed_forms():
    rng = np.random.default_rng(21)
    x = O.f32_to_bf16(rng.standard_normal((7, 512)).astype(np.float32) * 3)
    w = O.f32_to_bf16(1 + 0.2 * rng.standard_normal(512).astype(np.float32))
    got, none = O.rms_norm(x, w, 1e-6)
    assert none is None
    xt, wt = P.to_torch(x).double(), P.to_torch(w).double()
    want = torch.nn.functional.rms_norm(xt, (512,), wt, 1e-6)
    assert _ulps(got, P.from_torch(want.float().to(torch.bfloat16))) <= 1
    # a wrong eps placement or a sum instead of a mean shows on small rows
    tiny = O.f32_to_bf16(np.full((1, 128), 1e-3, dtype=np.float32))
    got_t, _ = O.rms_norm(tiny, O.f32_to_bf16(np.ones(128, dtype=np.float32)), 1e-6)
    t = float(O.bf16_to_f32(tiny)[0, 0])
    assert np.allclose(O.bf16_to_f32(got_t), t / np.sqrt(t * t + 1e-6), rtol=1e-2)
    # constant row: out == sign(c) * weight; scale invariance
    c = O.f32_to_bf16(np.full((1, 512), -4.0, dtype=np.float32))
    got_c, _ = O.rms_norm(c, w, 0.0)
    assert np.array_equal(got_c[0], O.f32_to_bf16(-O.bf16_to_f32(w)))
    x4 = O.f32_to_bf16(O.bf16_to_f32(x) * 4.0)
    assert np.array_equal(O.rms_norm(x4, w, 0.0)[0], O.rms_norm(x, w, 0.0)[0])


def test_rms_norm_with_residual_is_norm_of_the_bf16_sum():
    rng = np.random.default_rng(22)
    x = O.f32_to_bf16(rng.standard_normal((5, 256)).astype(np.float32))
    r = O.f32_to_bf16(rng.standard_normal((5, 256)).astype(np.float32) * 2)
    w = O.f32_to_bf16(1 + 0.1 * rng.standard_normal(256).astype(np.float32))
    got, new_r = O.rms_norm(x, w, 1e-6, residual=r)
    want_r = P.from_torch(P.to_torch(x) + P.to_torch(r))  # torch's own bf16 tensor add
    assert np.array_equal(new_r, want_r)
    assert np.array_equal(got, O.rms_norm(want_r, w, 1e-6)[0])
    assert np.array_equal(O.rms_norm(r, w, 1e-6, residual=x)[0], got)  # the add commutes


def test_qkv_norm_split_against_torch():
    rng = np.random.default_rng(23)
    B, Hq, Hkv = 3, 4, 2
    qkv = O.f32_to_bf16(rng.standard_normal((B, (Hq + 2 * Hkv) * D)).astype(np.float32) * 2)
    qw = O.f32_to_bf16(1 + 0.3 * rng.standard_normal(D).astype(np.float32))
    kw = O.f32_to_bf16(1 + 0.3 * rng.standard_normal(D).astype(np.float32))
    q, k, v = O.qkv_norm_split(qkv, qw, kw, 1e-6, Hq, Hkv)
    t = P.to_torch(qkv).double()
    tq, tk, tv = t.split((Hq * D, Hkv * D, Hkv * D), dim=-1)
    wq = torch.nn.functional.rms_norm(tq.reshape(B, Hq, D), (D,), P.to_torch(qw).double(), 1e-6)
    wk = torch.nn.functional.rms_norm(tk.reshape(B, Hkv, D), (D,), P.to_torch(kw).double(), 1e-6)
    assert q.shape == (B, Hq, D) and k.shape == (B, Hkv, D) and v.shape == (B, Hkv, D)
    assert _ulps(q, P.from_torch(wq.float().to(torch.bfloat16))) <= 1
    assert _ulps(k, P.from_torch(wk.float().to(torch.bfloat16))) <= 1
    assert np.array_equal(v, P.from_torch(tv.reshape(B, Hkv, D).float().to(torch.bfloat16)))
    # q and k use their own weights
    assert not np.array_equal(O.qkv_norm_split(qkv, kw, qw, 1e-6, Hq, Hkv)[0], q)


@pytest.mark.parametrize("act", ["silu", "gelu", "relu"])
def test_gated_act_against_torch_bf16_ops(act):
    rng = np.random.default_rng(24)
    g = O.f32_to_bf16(rng.standard_normal((4, 64)).astype(np.float32) * 3)
    u = O.f32_to_bf16(rng.standard_normal((4, 64)).astype(np.float32) * 2)
    fn = {"silu": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu, "relu": torch.relu}[act]
    want = fn(P.to_torch(g)) * P.to_torch(u)  # two bf16 tensor operations
    got = O.gated_act(g, u, act)
    assert _ulps(got, P.from_torch(want)) <= 1
    # closed forms: act(0) = 0; large positive gates pass up through
    z = O.gated_act(O.f32_to_bf16(np.zeros((1, 8), dtype=np.float32)), u[:1, :8], act)
    assert np.all(O.bf16_to_f32(z) == 0)
    big = O.f32_to_bf16(np.full((1, 8), 32.0, dtype=np.float32))
    assert np.array_equal(O.gated_act(big, u[:1, :8], act), O.f32_to_bf16(32.0 * O.bf16_to_f32(u[:1, :8])))
    with pytest.raises(ValueError):
        O.gated_act(g, u, "tanh")


@pytest.mark.parametrize("act", ["silu", "gelu", "relu"])
def test_layer_rows_in_float16_against_torch(act):
    """The same three functions inside element_format("f16"): torch's own float16
    tensor operations (computed in fp32, rounded once per operation) are the pin."""
    rng = np.random.default_rng(25)
    with O.element_format("f16"):
        x = O.f32_to_elem(rng.standard_normal((6, 256)).astype(np.float32) * 3)
        r = O.f32_to_elem(rng.standard_normal((6, 256)).astype(np.float32) * 2)
        w = O.f32_to_elem(1 + 0.2 * rng.standard_normal(256).astype(np.float32))
        assert P.to_torch(x).dtype == torch.float16
        got, new_r = O.rms_norm(x, w, 1e-6, residual=r)
        want_r = P.to_torch(x) + P.to_torch(r)              # one float16 tensor add
        assert np.array_equal(new_r, P.from_torch(want_r))
        want = torch.nn.functional.rms_norm(want_r.double(), (256,), P.to_torch(w).double(), 1e-6)
        assert _ulps_elem(got, P.from_torch(want.float().to(torch.float16))) <= 1
        g = O.f32_to_elem(rng.standard_normal((4, 64)).astype(np.float32) * 3)
        u = O.f32_to_elem(rng.standard_normal((4, 64)).astype(np.float32) * 2)
        fn = {"silu": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu, "relu": torch.relu}[act]
        want_g = fn(P.to_torch(g)) * P.to_torch(u)          # two float16 tensor operations
        # torch evaluates gelu in fp32, where 1 + erf(g / sqrt 2) cancels for g < -2: its own error (1e-4
        # relative) shows at float16's 11 bits, the oracle's float64 does not have it
        assert _ulps_elem(O.gated_act(g, u, act), P.from_torch(want_g)) <= (2 if act == "gelu" else 1)
        # the format matters: the same bits read as bf16 give another answer
        assert not np.array_equal(O.rms_norm(x, w, 1e-6)[0], _as_bf16(lambda: O.rms_norm(x, w, 1e-6)[0]))


def _as_bf16(fn):
    with O.element_format("bf16"):
        return fn()


def _ulps_elem(a_bits, b_bits):
    def key(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, 0x8000 - b, b)

    near = np.abs(O.elem_to_f32(a_bits).astype(np.float64) - O.elem_to_f32(b_bits)) <= 1e-6
    return int(np.where(near, 0, np.abs(key(a_bits) - key(b_bits))).max())
