"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py):
the oracle must keep reproducing them on CPU, and the HIP path must match them
on the GPU."""
import glob
import os

import numpy as np
import pytest

from oracle import blocktopk_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))


def load(path):
    with np.load(path, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def test_fixtures_exist():
    assert len(FIXTURES) >= 5


@pytest.mark.parametrize("path", FIXTURES, ids=lambda p: os.path.basename(p))
def test_oracle_reproduces_golden(path):
    f = load(path)
    kv, kbar = f["kv_cache"].copy(), f["kbar"].copy()
    res = O.decode_step(f["q"], f["k"], f["v"], kv, kbar, f["page_indices"], f["page_indptr"], f["last_page_len"], int(f["topk"]),
                        sink_pages=int(f["sink_pages"]), local_tokens=int(f["local_tokens"]),
                        first_page_offset=int(f["first_page_offset"]))
    assert np.array_equal(kv, f["exp_kv_cache"]) and np.array_equal(kbar, f["exp_kbar"])
    assert np.array_equal(res["sel_pages"], f["exp_sel_pages"]) and np.array_equal(res["sel_count"], f["exp_sel_count"])
    assert np.allclose(res["out"], f["exp_out"], rtol=1e-12, atol=1e-14)
    assert np.allclose(res["lse"], f["exp_lse"], rtol=1e-12)
    dense, dense_lse = O.dense_paged_decode(f["q"], kv, f["page_indices"], f["page_indptr"], f["last_page_len"],
                                            first_page_offset=int(f["first_page_offset"]))
    assert np.allclose(dense, f["exp_dense_out"], rtol=1e-12, atol=1e-14)
    assert np.allclose(dense_lse, f["exp_dense_lse"], rtol=1e-12)


def test_ties_fixture_selects_lowest_indices():
    f = load(os.path.join(HERE, "golden", "ties.npz"))
    pages = f["page_indices"]
    assert f["exp_sel_pages"][0, 0, :3].tolist() == pages[:3].tolist()
    assert f["exp_sel_pages"][0, 0, 3] == pages[-1]


@pytest.mark.gpu
@pytest.mark.parametrize("path", FIXTURES, ids=lambda p: os.path.basename(p))
def test_hip_path_matches_golden(path):
    import torch

    from kinetics_amd import ops
    from tests import problems as P

    f = load(path)
    dev = "cuda"
    q, k, v, kv, kbar = (P.to_torch(f[n], dev) for n in ("q", "k", "v", "kv_cache", "kbar"))
    idx, ptr, last = (P.int_tensor(f[n], dev) for n in ("page_indices", "page_indptr", "last_page_len"))
    topk, sink, local, offset = int(f["topk"]), int(f["sink_pages"]), int(f["local_tokens"]), int(f["first_page_offset"])
    B, Hkv = q.shape[0], kv.shape[3]
    sel = torch.empty(B, Hkv, f["exp_sel_pages"].shape[2], dtype=torch.int32, device=dev)
    assert sel.shape[2] == ops.sel_list_capacity(topk, sink, local)
    cnt = torch.empty(B, Hkv, dtype=torch.int32, device=dev)
    lse = torch.empty(B, q.shape[1], dtype=torch.float32, device=dev)
    ops.check_page_table(idx, ptr, last, P.PAGE_SIZE, kv.shape[0])
    ops.append_paged_kv(k, v, kv, kbar, idx, ptr, last)
    ops.block_score_topk(q, kbar, idx, ptr, last, topk, sel, cnt, sink_pages=sink, local_tokens=local)
    out = ops.sparse_paged_decode(q, kv, sel, cnt, last, lse=lse, first_page_offset=offset)
    dense = ops.dense_paged_decode(q, kv, idx, ptr, last, int(np.diff(f["page_indptr"]).max()), first_page_offset=offset)
    torch.cuda.synchronize()
    assert np.array_equal(P.from_torch(kv), f["exp_kv_cache"])          # bit-exact bytes
    assert np.array_equal(P.from_torch(kbar), f["exp_kbar"])
    assert np.array_equal(cnt.cpu().numpy(), f["exp_sel_count"])
    assert np.array_equal(sel.cpu().numpy(), f["exp_sel_pages"])          # indices, order and padding
    for got, want in ((out, f["exp_out"]), (dense, f["exp_dense_out"])):
        err = np.abs(got.float().cpu().numpy() - want)
        assert np.all(err <= 2e-2 + 2e-2 * np.abs(want))                  # bf16 output tolerance
    assert np.allclose(lse.cpu().numpy(), f["exp_lse"], rtol=1e-4, atol=1e-4)
