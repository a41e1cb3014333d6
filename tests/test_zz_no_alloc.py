"""The decode step's entry point that allocates nothing
(kin_blocktopk_decode_step_static: the workspace through which workgroups share a
list = an array inside the library's device code) against the existing entry point it is a variant of
(kin_blocktopk_decode_step with a caller workspace), through the C ABI: cache
bytes, page lists and attention output bit-equal, on calls in a row that share
the array -- the second with a smaller input, so the first call's keys are still
lying behind it -- and against the oracle.
"""
import ctypes

import numpy as np
import pytest
import torch

from oracle import blocktopk_oracle as O
from tests import problems as P

pytestmark = pytest.mark.gpu

PS = P.PAGE_SIZE
DEV = "cuda"


class Gpu:
    def __init__(self, pb, cap):
        self.q, self.k, self.v = (P.to_torch(x, DEV) for x in (pb.q, pb.k, pb.v))
        self.kv, self.kbar = P.to_torch(pb.kv_cache, DEV), P.to_torch(pb.kbar, DEV)
        self.indices, self.indptr, self.last = (P.int_tensor(x, DEV) for x in (pb.page_indices, pb.page_indptr, pb.last_page_len))
        self.sel = torch.full((pb.B, pb.Hkv, cap), -7, dtype=torch.int32, device=DEV)
        self.cnt = torch.full((pb.B, pb.Hkv), -7, dtype=torch.int32, device=DEV)
        self.out = torch.full((pb.B, pb.Hq, P.HEAD_DIM), float("nan"), dtype=torch.bfloat16, device=DEV)
        self.lse = torch.full((pb.B, pb.Hq), float("nan"), dtype=torch.float32, device=DEV)


def _both_ways(ops, pb, sink, local, what, must_split):
    cap = ops.sel_list_capacity(pb.topk, sink, local)
    need = ops.step_workspace_bytes(pb.B, pb.Hkv, pb.kbar.shape[2])
    assert (need > 0) == must_split, what
    a, b = Gpu(pb, cap), Gpu(pb, cap)
    ws = torch.full((max(need, 16),), 0x5A, dtype=torch.uint8, device=DEV)
    ops.blocktopk_decode_step(a.q, a.k, a.v, a.kv, a.kbar, a.indices, a.indptr, a.last, pb.topk, out=a.out, lse=a.lse,
                              sel_pages=a.sel, sel_count=a.cnt, sink_pages=sink, local_tokens=local, workspace=ws)
    ops.blocktopk_decode_step(b.q, b.k, b.v, b.kv, b.kbar, b.indices, b.indptr, b.last, pb.topk, out=b.out, lse=b.lse,
                              sel_pages=b.sel, sel_count=b.cnt, sink_pages=sink, local_tokens=local, static_scratch=True)
    torch.cuda.synchronize()
    assert torch.equal(a.kv, b.kv) and torch.equal(a.kbar, b.kbar), f"{what}: cache bytes differ"
    assert torch.equal(a.cnt, b.cnt) and torch.equal(a.sel, b.sel), f"{what}: page lists differ"
    assert torch.equal(a.out.view(torch.int16), b.out.view(torch.int16)), f"{what}: outputs differ"
    assert torch.equal(a.lse, b.lse), f"{what}: lse differs"
    # and both are right: append bit-exact, list lengths exact, output within the contract of the oracle on the GPU's lists
    kv, kbar = pb.kv_cache.copy(), pb.kbar.copy()
    res = O.decode_step(pb.q, pb.k, pb.v, kv, kbar, pb.page_indices, pb.page_indptr, pb.last_page_len, pb.topk,
                        sink_pages=sink, local_tokens=local)
    assert np.array_equal(P.from_torch(b.kv), kv) and np.array_equal(P.from_torch(b.kbar), kbar), what
    assert np.array_equal(b.cnt.cpu().numpy(), res["sel_count"]), what
    want, _ = O.sparse_paged_decode(pb.q, kv, b.sel.cpu().numpy(), res["sel_count"], pb.last_page_len)
    got = b.out.float().cpu().numpy().astype(np.float64)
    err = np.abs(got - want)
    assert np.all(err <= 2e-2 + 2e-2 * np.abs(want)), f"{what}: max err {err.max()}"


def test_static_scratch_step_equals_workspace_step():
    from kinetics_amd import _lib, ops

    lib = _lib.load()
    assert lib.kin_static_scratch_bytes() == 4 * 1024 * 1024 + 64 * 1024
    # two calls in a row on the same array, the second smaller (fewer and shorter lists): the
    # first call's keys and counters are what the second finds there
    big = P.make_problem(9101, [PS * 2500 + 3, PS * 2100 + 16, 5, 0, PS * 300 + 1], num_kv_heads=2, group=4, topk=40)
    _both_ways(ops, big, sink=1, local=17, what="first call (5 sequences x 2 KV heads, up to 2501 pages)", must_split=True)
    small = P.make_problem(9102, [PS * 2048 + 9, 70], num_kv_heads=1, group=8, topk=64)
    _both_ways(ops, small, sink=0, local=1, what="second call (2 sequences, up to 2049 pages)", must_split=True)
    # a shape with lists for more than half the CUs shares nothing between workgroups and never touches the array
    plain = P.make_problem(9103, [PS * 40 + 1] * 69 + [3], num_kv_heads=2, group=2, topk=8)
    _both_ways(ops, plain, sink=0, local=1, what="third call (one workgroup per list)", must_split=False)
    # few lists with long page lists: larger teams, more partial results (8 lists x 32 parts x 16 heads: 2.1 MB)
    parts = P.make_problem(9104, [PS * 400 + 1, PS * 300 + 16, 9], num_kv_heads=2, group=4, topk=150)
    _both_ways(ops, parts, sink=1, local=20, what="fourth call (split attention)", must_split=True)
    full = P.make_problem(9105, [PS * 1300 + 5] * 4, num_kv_heads=2, group=16, topk=1100)
    _both_ways(ops, full, sink=0, local=1, what="fifth call (split attention, 16 heads per list)", must_split=True)
    # a few lists more than CUs: the 24 lists beyond the first 256 in teams
    tail = P.make_problem(9107, [PS * 110 + 3] * 139 + [7], num_kv_heads=2, group=4, topk=100)
    _both_ways(ops, tail, sink=0, local=1, what="call with 280 lists (teams for the last 24)", must_split=True)
    # and the first shape once more after them
    _both_ways(ops, big, sink=0, local=33, what="sixth call (first shape again)", must_split=True)


def test_static_scratch_step_takes_no_device_memory():
    """Free device memory as the driver reports it is the same before and after calls of the entry point,
    with torch's caching allocator out of the picture: every tensor exists before the first reading.
    (One call comes before the first reading: the runtime loads a kernel's code the first time it is
    launched, which is the runtime's memory, not the entry point's.)"""
    from kinetics_amd import ops

    pb = P.make_problem(9106, [PS * 2200 + 3, PS * 900 + 16, 5], num_kv_heads=2, group=4, topk=40)
    g = Gpu(pb, ops.sel_list_capacity(pb.topk, 0, 1))

    def call():
        ops.blocktopk_decode_step(g.q, g.k, g.v, g.kv, g.kbar, g.indices, g.indptr, g.last, pb.topk, out=g.out, lse=g.lse,
                                  sel_pages=g.sel, sel_count=g.cnt, static_scratch=True)

    call()
    torch.cuda.synchronize()
    reserved0 = torch.cuda.memory_reserved()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(5):
        call()
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert torch.cuda.memory_reserved() == reserved0, "torch allocated device memory during the calls"
    assert free1 == free0, f"free device memory went from {free0} to {free1} bytes across kin_blocktopk_decode_step_static"


def test_static_scratch_step_rejects_sizes_beyond_the_array():
    from kinetics_amd import _lib

    lib = _lib.load()
    # 64 lists of 16384 candidate pages want 4 MiB of keys and 0.5 MB of partial results: more than the array holds.  The size
    # test comes first, from the dimensions alone: no pointer is looked at.
    assert lib.kin_step_workspace_bytes(64, 1, 16384) > lib.kin_static_scratch_bytes()
    null = ctypes.c_void_p(None)
    st = lib.kin_blocktopk_decode_step_static(null, null, null, null, null, null, null, null, 128, 0, 1, null, null, null, null,
                                              64, 4, 1, 128, 16, 1 << 20, 16384, 0, 0, 0.0, null, 0, null, null)
    assert st == _lib.KIN_ERR_WORKSPACE
    msg = lib.kin_last_error().decode()
    assert "kin_blocktopk_decode_step_static" in msg and "scratch" in msg
    with pytest.raises(_lib.KineticsError):
        _lib.check(st)
