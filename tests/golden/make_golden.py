#!/usr/bin/env python3
"""Writes the golden fixtures in this directory: small seeded decode problems
(inputs) and the results the oracle gives for them (expected outputs).

The reference repository holds no tests, golden vectors or fixtures for this
path, and its implementation cannot run here (it imports flashinfer), so these
vectors come from ``oracle/blocktopk_oracle.py``, which tests/test_oracle.py
pins against library routines and closed forms.  They freeze the oracle's
behaviour (a later change to it shows up as a diff) and give the HIP path a
fixed target that does not depend on numpy's random streams.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import blocktopk_oracle as O  # noqa: E402
from tests import problems as P  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
PS = P.PAGE_SIZE

CASES = {
    # name: (seed, lengths, num_kv_heads, group, topk, table, all_equal_kbar, sink_pages, local_tokens, first_page_offset)
    "basic": (1001, [PS * 5 + 3, PS * 2, 7], 1, 4, 2, "random", False, 0, 1, 0),
    "hkv2_fills_page": (1002, [PS * 4 + 16, PS * 3 + 1], 2, 2, 2, "random", False, 0, 1, 0),
    "ties": (1003, [PS * 8 + 2], 1, 4, 3, "random", True, 0, 1, 0),
    "sink_local": (1004, [PS * 9 + 5, PS * 3 + 1], 1, 4, 2, "random", False, 1, 17, 0),
    # LiteSys' geometry: 4 sink tokens in slots 12..15 of the first page, 20 local tokens
    "sink_local_offset12": (1005, [PS * 11 + 7, PS * 6, 14], 2, 2, 3, "random", False, 1, 20, 12),
    # head rows of 64 elements (an eleventh entry: the head dimension; 128 when absent)
    "head_dim_64": (1006, [PS * 7 + 9, PS * 2 + 16, 5], 2, 4, 3, "random", False, 1, 17, 0, 64),
}


def make(name):
    seed, lengths, hkv, group, topk, table, equal, sink, local, offset = CASES[name][:10]
    with P.head_dim(CASES[name][10] if len(CASES[name]) > 10 else 128):
        pb = P.make_problem(seed, lengths, num_kv_heads=hkv, group=group, topk=topk, table=table, extra_pages=1, kbar_slack=1)
    if equal:
        pb.kbar[:] = pb.kbar[0, 0, 0]
    inputs = dict(q=pb.q, k=pb.k, v=pb.v, kv_cache=pb.kv_cache.copy(), kbar=pb.kbar.copy(),
                  page_indices=pb.page_indices, page_indptr=pb.page_indptr, last_page_len=pb.last_page_len,
                  topk=np.int32(topk), sink_pages=np.int32(sink), local_tokens=np.int32(local),
                  first_page_offset=np.int32(offset))
    res = O.decode_step(pb.q, pb.k, pb.v, pb.kv_cache, pb.kbar, pb.page_indices, pb.page_indptr, pb.last_page_len, topk,
                        sink_pages=sink, local_tokens=local, first_page_offset=offset)
    dense, dense_lse = O.dense_paged_decode(pb.q, pb.kv_cache, pb.page_indices, pb.page_indptr, pb.last_page_len,
                                            first_page_offset=offset)
    expected = dict(exp_kv_cache=pb.kv_cache, exp_kbar=pb.kbar, exp_sel_pages=res["sel_pages"],
                    exp_sel_count=res["sel_count"], exp_out=res["out"], exp_lse=res["lse"], exp_dense_out=dense,
                    exp_dense_lse=dense_lse)
    np.savez_compressed(os.path.join(HERE, f"{name}.npz"), **inputs, **expected)


if __name__ == "__main__":
    for n in (sys.argv[1:] or CASES):   # all of them, or the ones named
        make(n)
        print("wrote", n, os.path.getsize(os.path.join(HERE, f"{n}.npz")), "bytes")
