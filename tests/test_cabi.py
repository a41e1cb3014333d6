"""The C-ABI library without a GPU: it loads, exports every symbol the header
declares, and rejects bad arguments with the documented status codes before
touching the device."""
import ctypes
import re
from pathlib import Path

import pytest

from kinetics_amd import _lib

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "kinetics_amd.h"

A = 0x1000  # a non-null, 16-byte aligned dummy address; never dereferenced on these paths


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(kin_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree(lib):
    syms = declared_symbols()
    assert len(syms) >= 11
    assert sorted(_lib.SIGNATURES) == syms
    for s in syms:
        assert hasattr(lib, s), f"{s} is declared in the header but not exported"


def test_version_and_status_strings(lib):
    assert lib.kin_version() >= 100
    assert lib.kin_status_string(0) == b"KIN_OK"
    assert lib.kin_status_string(_lib.KIN_ERR_BAD_SHAPE) == b"KIN_ERR_BAD_SHAPE"
    assert lib.kin_status_string(99) == b"KIN_ERR_UNKNOWN"


def append(lib, k=A, v=A, kv=A, kbar=A, idx=A, ptr=A, last=A, B=2, Hkv=1, D=128, ps=16, P=8, kp=4, slots=None, ns=0):
    return lib.kin_append_paged_kv(k, v, kv, kbar, idx, ptr, last, B, Hkv, D, ps, P, kp, slots, ns, None)


def test_append_argument_errors(lib):
    assert append(lib, k=None) == _lib.KIN_ERR_NULL_POINTER
    assert append(lib, ptr=None) == _lib.KIN_ERR_NULL_POINTER
    assert append(lib, B=-1) == _lib.KIN_ERR_BAD_SHAPE
    assert append(lib, Hkv=0) == _lib.KIN_ERR_BAD_SHAPE
    assert append(lib, P=0) == _lib.KIN_ERR_BAD_SHAPE
    assert append(lib, kp=0) == _lib.KIN_ERR_BAD_SHAPE
    assert append(lib, D=96) == _lib.KIN_ERR_UNSUPPORTED
    assert b"64 and 128" in lib.kin_last_error()
    assert append(lib, D=64, B=0) == _lib.KIN_OK              # the page path is built for head rows of 64 and 128
    assert append(lib, ps=24) == _lib.KIN_ERR_UNSUPPORTED
    assert append(lib, ps=256) == _lib.KIN_ERR_UNSUPPORTED
    assert append(lib, ps=32, B=0) == _lib.KIN_OK and append(lib, ps=64, B=0) == _lib.KIN_OK and append(lib, ps=128, B=0) == _lib.KIN_OK
    assert append(lib, kv=A + 2) == _lib.KIN_ERR_MISALIGNED
    assert b"kv_cache" in lib.kin_last_error()
    assert append(lib, B=0) == _lib.KIN_OK  # nothing to do, nothing launched
    assert append(lib, slots=A, ns=0) == _lib.KIN_ERR_BAD_SHAPE       # a slot table without slots
    assert b"num_slots" in lib.kin_last_error()
    assert append(lib, slots=A, ns=4, B=0) == _lib.KIN_OK


def test_ragged_append_argument_errors(lib):
    def ragged(k=A, ind=A, B=2, nnz=10, mx=10, kv=A):
        return lib.kin_append_paged_kv_ragged(k, A, ind, kv, A, A, A, A, B, nnz, mx, 1, 128, 16, 8, 4, None, 0, None)

    assert ragged(k=None) == _lib.KIN_ERR_NULL_POINTER
    assert ragged(ind=None) == _lib.KIN_ERR_NULL_POINTER
    assert ragged(nnz=-1) == _lib.KIN_ERR_BAD_SHAPE
    assert ragged(nnz=4, mx=5) == _lib.KIN_ERR_BAD_SHAPE
    assert ragged(kv=A + 4) == _lib.KIN_ERR_MISALIGNED
    assert ragged(nnz=0, mx=0) == _lib.KIN_OK
    assert ragged(B=0) == _lib.KIN_OK


def select(lib, q=A, kbar=A, idx=A, ptr=A, last=A, topk=4, sel=A, cnt=A, B=2, Hq=4, Hkv=1, D=128, kp=64, stride=5, sink=0,
           local=1, ps=16, slots=None, ns=0):
    return lib.kin_block_score_topk(q, kbar, idx, ptr, last, topk, sink, local, sel, cnt, None, None, B, Hq, Hkv, D, ps, kp,
                                    stride, None, 0, slots, ns, None)


def test_select_argument_errors(lib):
    assert select(lib, q=None) == _lib.KIN_ERR_NULL_POINTER
    assert select(lib, cnt=None) == _lib.KIN_ERR_NULL_POINTER
    assert select(lib, last=None) == _lib.KIN_ERR_NULL_POINTER
    assert select(lib, topk=-1) == _lib.KIN_ERR_BAD_SHAPE
    assert select(lib, stride=4) == _lib.KIN_ERR_BAD_SHAPE          # no room for the last page
    assert select(lib, stride=5, sink=1) == _lib.KIN_ERR_BAD_SHAPE  # nor for a sink page on top
    assert select(lib, stride=5, local=2) == _lib.KIN_ERR_BAD_SHAPE  # 2 local tokens can span 2 pages
    assert b"kin_sel_list_capacity" in lib.kin_last_error()
    assert select(lib, local=0) == _lib.KIN_ERR_BAD_SHAPE           # the open page is always attended
    assert select(lib, sink=-1) == _lib.KIN_ERR_BAD_SHAPE
    assert select(lib, stride=200, local=1010) == _lib.KIN_ERR_BAD_SHAPE
    assert select(lib, Hq=5, Hkv=2) == _lib.KIN_ERR_BAD_SHAPE
    assert select(lib, Hq=32, Hkv=1) == _lib.KIN_ERR_UNSUPPORTED    # group 32 > 16
    assert select(lib, topk=4096, stride=4097) == _lib.KIN_ERR_UNSUPPORTED
    assert select(lib, kp=20000) == _lib.KIN_ERR_UNSUPPORTED
    assert select(lib, kbar=A + 8) == _lib.KIN_ERR_MISALIGNED
    assert select(lib, ps=48) == _lib.KIN_ERR_UNSUPPORTED
    assert select(lib, B=0) == _lib.KIN_OK and select(lib, B=0, ps=64) == _lib.KIN_OK
    assert select(lib, slots=A, ns=-1) == _lib.KIN_ERR_BAD_SHAPE


def sparse(lib, q=A, kv=A, sel=A, cnt=A, last=A, out=A, ws=None, wsb=0, B=2, Hq=4, Hkv=1, D=128, ps=16, P=8,
           stride=5, splits=1, offset=0):
    return lib.kin_sparse_paged_decode(q, kv, sel, cnt, last, out, None, ws, wsb, B, Hq, Hkv, D, ps, P, stride, offset, 0.0,
                                       splits, None)


def test_decode_argument_errors(lib):
    assert sparse(lib, out=None) == _lib.KIN_ERR_NULL_POINTER
    assert sparse(lib, sel=None) == _lib.KIN_ERR_NULL_POINTER
    assert sparse(lib, stride=0) == _lib.KIN_ERR_BAD_SHAPE
    assert sparse(lib, splits=-1) == _lib.KIN_ERR_BAD_SHAPE
    assert sparse(lib, offset=16) == _lib.KIN_ERR_BAD_SHAPE
    assert sparse(lib, offset=-1) == _lib.KIN_ERR_BAD_SHAPE
    assert sparse(lib, D=256) == _lib.KIN_ERR_UNSUPPORTED
    assert sparse(lib, q=A + 4) == _lib.KIN_ERR_MISALIGNED
    # split-K without (enough) workspace
    assert sparse(lib, splits=3) == _lib.KIN_ERR_WORKSPACE
    need = lib.kin_decode_workspace_bytes(2, 4, 1, 128, 5, 3)
    assert need == 2 * 4 * 3 * 129 * 4
    assert sparse(lib, splits=3, ws=A, wsb=need - 1) == _lib.KIN_ERR_WORKSPACE
    assert b"workspace" in lib.kin_last_error()
    assert sparse(lib, B=0) == _lib.KIN_OK
    dense = lib.kin_dense_paged_decode(A, A, None, A, A, A, None, None, 0, 2, 4, 1, 128, 16, 8, 9, 0, 0.0, 1, None)
    assert dense == _lib.KIN_ERR_NULL_POINTER
    dense = lib.kin_dense_paged_decode(A, A, A, A, A, A, None, None, 0, 2, 4, 1, 128, 16, 8, 0, 0, 0.0, 1, None)
    assert dense == _lib.KIN_ERR_BAD_SHAPE
    dense = lib.kin_dense_paged_decode(A, A, A, A, A, A, None, None, 0, 2, 4, 1, 128, 16, 8, 9, 16, 0.0, 1, None)
    assert dense == _lib.KIN_ERR_BAD_SHAPE


def step(lib, q=A, k=A, v=A, kv=A, kbar=A, idx=A, ptr=A, last=A, topk=4, sink=0, local=1, sel=None, cnt=None, out=A, B=2,
         Hq=4, Hkv=1, D=128, ps=16, P=8, kp=64, stride=0, offset=0, slots=None, ns=0):
    return lib.kin_blocktopk_decode_step(q, k, v, kv, kbar, idx, ptr, last, topk, sink, local, sel, cnt, out, None, B, Hq, Hkv,
                                         D, ps, P, kp, stride, offset, 0.0, None, 0, slots, ns, None, None)


def test_step_argument_errors(lib):
    assert step(lib, kbar=None) == _lib.KIN_ERR_NULL_POINTER
    assert step(lib, v=None) == _lib.KIN_ERR_NULL_POINTER            # k without v
    assert step(lib, topk=-1) == _lib.KIN_ERR_BAD_SHAPE
    assert step(lib, local=0) == _lib.KIN_ERR_BAD_SHAPE
    assert step(lib, offset=16) == _lib.KIN_ERR_BAD_SHAPE
    assert step(lib, offset=12) == _lib.KIN_ERR_BAD_SHAPE            # a padded first page must be a sink page
    assert b"sink_pages" in lib.kin_last_error()
    assert step(lib, sel=A, cnt=A, stride=4) == _lib.KIN_ERR_BAD_SHAPE
    assert step(lib, sel=A, stride=5) == _lib.KIN_ERR_NULL_POINTER   # list without its count
    assert step(lib, topk=4096) == _lib.KIN_ERR_UNSUPPORTED
    assert step(lib, out=A + 2) == _lib.KIN_ERR_MISALIGNED
    assert step(lib, B=0, sink=1, offset=12) == _lib.KIN_OK
    assert step(lib, slots=A, ns=0) == _lib.KIN_ERR_BAD_SHAPE


def test_token_topk_argument_errors(lib):
    def tok(q=A, topk=8, sink=4, local=1, offset=0, sel=None, cnt=None, ws=A, wsb=1 << 20, B=2, Hq=4, Hkv=1, P=8, mp=4,
            stride=0, D=128):
        return lib.kin_token_topk_decode(q, A, A, A, A, topk, sink, local, offset, sel, cnt, A, None, ws, wsb, B, Hq, Hkv,
                                         D, 16, P, mp, stride, 0.0, None)

    assert tok(q=None) == _lib.KIN_ERR_NULL_POINTER
    assert tok(topk=-1) == _lib.KIN_ERR_BAD_SHAPE
    assert tok(offset=16) == _lib.KIN_ERR_BAD_SHAPE
    assert tok(mp=0) == _lib.KIN_ERR_BAD_SHAPE
    assert tok(topk=5000) == _lib.KIN_ERR_UNSUPPORTED
    assert tok(local=2000) == _lib.KIN_ERR_UNSUPPORTED
    assert tok(D=96) == _lib.KIN_ERR_UNSUPPORTED                      # head rows of 64 and 128 elements only
    assert b"head_dim=96" in lib.kin_last_error()
    assert tok(D=64, B=0) == _lib.KIN_OK
    assert tok(sel=A, cnt=A, stride=12) == _lib.KIN_ERR_BAD_SHAPE      # 8 + 4 + 1 entries needed
    assert tok(sel=A, stride=13) == _lib.KIN_ERR_NULL_POINTER
    assert lib.kin_token_topk_workspace_bytes(2, 1, 4) == 256 + 2 * 4 * 16 * 4  # arrival counters + keys
    assert tok(wsb=2 * 4 * 16 * 4 - 1) == _lib.KIN_ERR_WORKSPACE
    assert tok(ws=None) == _lib.KIN_ERR_WORKSPACE
    assert tok(P=1 << 28) == _lib.KIN_ERR_UNSUPPORTED                  # token ids would not fit 31 bits
    assert tok(B=0) == _lib.KIN_OK


def test_strided_topk_argument_errors(lib):
    def strided(topk=2, block=16, stride=8, sel=None, cnt=None, wsb=1 << 20, B=2, mp=4, sel_stride=0):
        return lib.kin_strided_topk_decode(A, A, A, A, A, topk, block, stride, 4, 1, 0, sel, cnt, A, None, A, wsb, B, 4, 1,
                                           128, 16, 8, mp, sel_stride, 0.0, None)

    assert strided(block=0) == _lib.KIN_ERR_BAD_SHAPE
    assert strided(block=65) == _lib.KIN_ERR_BAD_SHAPE
    assert strided(stride=0) == _lib.KIN_ERR_BAD_SHAPE
    assert strided(topk=300) == _lib.KIN_ERR_UNSUPPORTED              # 300 * 16 tokens > 4096
    assert strided(sel=A, cnt=A, sel_stride=36) == _lib.KIN_ERR_BAD_SHAPE   # 2 * 16 + 4 + 1 entries needed
    assert lib.kin_strided_topk_workspace_bytes(2, 1, 4) == 256 + 2 * 2 * 4 * 16 * 4
    assert strided(wsb=2 * 2 * 4 * 16 * 4 - 1) == _lib.KIN_ERR_WORKSPACE
    assert strided(B=0) == _lib.KIN_OK


def test_layer_row_kernel_argument_errors(lib):
    def norm(x=A, res=None, w=A, out=A, rows=4, hidden=4096, xs=4096, os_=4096, eps=1e-6):
        return lib.kin_rms_norm(x, res, w, out, rows, hidden, xs, os_, eps, None)

    assert norm(x=None) == _lib.KIN_ERR_NULL_POINTER
    assert norm(w=None) == _lib.KIN_ERR_NULL_POINTER
    assert norm(rows=-1) == _lib.KIN_ERR_BAD_SHAPE
    assert norm(hidden=4100) == _lib.KIN_ERR_UNSUPPORTED   # not a multiple of 128
    assert norm(hidden=8704, xs=8704, os_=8704) == _lib.KIN_ERR_UNSUPPORTED  # above 8192
    assert norm(hidden=2176, xs=2176, os_=2176) == _lib.KIN_ERR_UNSUPPORTED  # multiple of 128 only, above 2048
    assert norm(xs=4000) == _lib.KIN_ERR_BAD_SHAPE         # stride below the row width
    assert norm(os_=4100) == _lib.KIN_ERR_BAD_SHAPE        # stride not a multiple of 8
    assert norm(eps=-1.0) == _lib.KIN_ERR_BAD_SHAPE
    assert norm(out=A + 4) == _lib.KIN_ERR_MISALIGNED
    assert norm(res=A + 8) == _lib.KIN_ERR_MISALIGNED
    assert norm(rows=0) == _lib.KIN_OK and norm(rows=0, hidden=128, xs=128, os_=128) == _lib.KIN_OK

    def split(qkv=A, stride=768, qw=A, kw=A, q=A, k=A, v=A, B=2, Hq=4, Hkv=1, D=128):
        return lib.kin_qkv_norm_split(qkv, stride, qw, kw, 1e-6, q, k, v, B, Hq, Hkv, D, None)

    assert split(kw=None) == _lib.KIN_ERR_NULL_POINTER
    assert split(v=None) == _lib.KIN_ERR_NULL_POINTER
    assert split(Hq=0) == _lib.KIN_ERR_BAD_SHAPE
    assert split(D=96) == _lib.KIN_ERR_UNSUPPORTED
    assert split(D=64, stride=384, B=0) == _lib.KIN_OK
    assert split(D=64, stride=380) == _lib.KIN_ERR_BAD_SHAPE   # narrower than (Hq + 2*Hkv) * 64
    assert split(stride=760) == _lib.KIN_ERR_BAD_SHAPE     # narrower than (Hq + 2*Hkv) * 128
    assert split(q=A + 2) == _lib.KIN_ERR_MISALIGNED
    assert split(B=0) == _lib.KIN_OK

    def gate(g=A, u=A, out=A, rows=2, inter=1536, gs=3072, us=3072, act=0):
        return lib.kin_gated_act(g, u, out, rows, inter, gs, us, act, None)

    assert gate(u=None) == _lib.KIN_ERR_NULL_POINTER
    assert gate(inter=1530) == _lib.KIN_ERR_BAD_SHAPE
    assert gate(gs=1000) == _lib.KIN_ERR_BAD_SHAPE
    assert gate(act=3) == _lib.KIN_ERR_UNSUPPORTED
    assert gate(g=A + 1) == _lib.KIN_ERR_MISALIGNED
    assert gate(rows=0) == _lib.KIN_OK


def test_sel_list_capacity(lib):
    assert lib.kin_sel_list_capacity(128, 0, 1) == 129               # the reference's k + 1
    assert lib.kin_sel_list_capacity(64, 1, 16) == 64 + 1 + 2
    assert lib.kin_sel_list_capacity(64, 1, 17) == 64 + 1 + 2
    assert lib.kin_sel_list_capacity(64, 1, 18) == 64 + 1 + 3
    assert lib.kin_sel_list_capacity(0, 0, 1) == 1
    assert lib.kin_sel_list_capacity(4, 0, 0) == 0


def test_auto_splits_policy(lib):
    assert lib.kin_decode_auto_splits(4096, 1, 129) == 1      # enough lists to fill the chip
    assert lib.kin_decode_auto_splits(8, 1, 65) > 1           # few lists: split along pages
    assert lib.kin_decode_auto_splits(8, 1, 3) == 1           # nothing to split
    assert lib.kin_decode_workspace_bytes(4096, 4, 1, 128, 129, 0) == 0


def test_auto_splits_policy_follows_the_lists(lib):
    """Few lists: about one workgroup per CU in total; between 256 and 768 lists long lists are
    split, shorter ones only just above a multiple of 256; from 768 lists on none; never fewer
    than 4 pages a split."""
    assert lib.kin_decode_auto_splits(8, 1, 2049) == 28
    assert lib.kin_decode_auto_splits(64, 1, 2049) == 4
    assert lib.kin_decode_auto_splits(4, 8, 257) == 7
    assert lib.kin_decode_auto_splits(256, 1, 2049) == 1
    assert lib.kin_decode_auto_splits(300, 1, 2049) == 7
    assert lib.kin_decode_auto_splits(300, 1, 513) == 4        # 44 lists more than one per CU
    assert lib.kin_decode_auto_splits(352, 1, 129) == 2 and lib.kin_decode_auto_splits(528, 1, 129) == 4
    assert lib.kin_decode_auto_splits(400, 1, 513) == 1 and lib.kin_decode_auto_splits(512, 1, 513) == 1
    assert lib.kin_decode_auto_splits(300, 1, 17) == 1         # too short to share
    assert lib.kin_decode_auto_splits(800, 1, 129) == 1
    assert lib.kin_decode_auto_splits(768, 1, 2049) == 1
    assert lib.kin_decode_auto_splits(1, 1, 1 << 20) == 64
    assert lib.kin_decode_auto_splits(8, 1, 17) == 4


def test_path_preference_rule():
    """prefer_fused_step: the single launch, except few lists of very long sequences with
    long page lists and long lists just above one list per CU."""
    from kinetics_amd import ops
    assert ops.prefer_fused_step(8, 1, 257, 64) and ops.prefer_fused_step(1, 8, 2049, 2048)
    assert ops.prefer_fused_step(64, 1, 2049, 512) and ops.prefer_fused_step(100, 1, 2049, 1024)
    assert ops.prefer_fused_step(8, 1, 8193, 128) and not ops.prefer_fused_step(8, 1, 8193, 256)
    assert not ops.prefer_fused_step(32, 1, 4097, 2048)
    assert ops.prefer_fused_step(256, 1, 1025, 64) and ops.prefer_fused_step(200, 1, 4097, 2048)
    assert ops.prefer_fused_step(300, 1, 2049, 768) and not ops.prefer_fused_step(300, 1, 2049, 1024)
    assert ops.prefer_fused_step(512, 8, 2049, 64) and ops.prefer_fused_step(4096, 1, 2049, 128)


def test_python_wrapper_maps_status_to_exceptions():
    with pytest.raises(ValueError, match="KIN_ERR_BAD_SHAPE"):
        _lib.check(_lib.load().kin_block_score_topk(A, A, A, A, A, -1, 0, 1, A, A, None, None, 2, 4, 1, 128, 16, 64, 5, None, 0, None, 0, None))
    with pytest.raises(_lib.KineticsError, match="KIN_ERR_WORKSPACE"):
        _lib.check(sparse(_lib.load(), splits=3))


def test_ops_reject_cpu_tensors_loudly():
    import torch

    from kinetics_amd import ops

    q = torch.zeros(2, 4, 128, dtype=torch.bfloat16)
    kv = torch.zeros(8, 2, 16, 1, 128, dtype=torch.bfloat16)
    i32 = torch.zeros(2, dtype=torch.int32)
    with pytest.raises(ValueError, match="GPU"):
        ops.sparse_paged_decode(q, kv, torch.zeros(2, 1, 5, dtype=torch.int32), torch.zeros(2, 1, dtype=torch.int32), i32)
    with pytest.raises(TypeError):
        ops.sparse_paged_decode(q, kv.float(), None, None, i32)


def test_custom_ops_are_registered_with_fake_kernels():
    import torch

    import kinetics_amd  # noqa: F401

    for name in ("append_paged_kv", "update_kv", "block_score_topk", "sparse_paged_decode", "dense_paged_decode",
                 "layer_norm", "qk_norm", "fused_layer_norm", "qkv_norm_split", "gated_act"):
        assert hasattr(torch.ops.kinetics, name)
    # the fake kernel gives shape/dtype without running anything (what torch.compile needs)
    q = torch.empty(3, 4, 128, dtype=torch.bfloat16, device="meta")
    kv = torch.empty(8, 2, 16, 1, 128, dtype=torch.bfloat16, device="meta")
    i = torch.empty(3, 1, 5, dtype=torch.int32, device="meta")
    c = torch.empty(3, 1, dtype=torch.int32, device="meta")
    l = torch.empty(3, dtype=torch.int32, device="meta")
    out = torch.ops.kinetics.sparse_paged_decode(q, kv, i, c, l, None, 0.0, 0)
    assert out.shape == q.shape and out.dtype == torch.bfloat16
    qkv = torch.empty(3, 6 * 128, dtype=torch.bfloat16, device="meta")
    w = torch.empty(128, dtype=torch.bfloat16, device="meta")
    fq, fk, fv = torch.ops.kinetics.qkv_norm_split(qkv, w, w, 1e-6, 4, 1)
    assert fq.shape == (3, 4, 128) and fk.shape == (3, 1, 128) and fv.shape == (3, 1, 128)
    assert torch.ops.kinetics.gated_act(qkv[:, :256], qkv[:, 256:512], "silu").shape == (3, 256)


def test_bench_byte_model_matches_the_documented_figures():
    """The algorithmic-bytes model behind the roofline figures: 1 576 960 B per
    sequence at the headline shape (k-bar stream + selected K/V + append + q/out +
    index write/read), 16 780 288 B for the dense baseline."""
    import bench

    ab = bench.algorithmic_bytes([32768 + 1] * 4096, 1, 4, 128)
    assert ab["step"] == 4096 * 1576960 == 6459228160
    assert ab["step"] // 4096 == 524288 + 1049088 + 512 + 2048 + 1024
    assert ab["dense"] == 4096 * 16780288
    assert ab["attention"] == 4096 * (1049088 + 2048 + 129 * 4)
    small = bench.algorithmic_bytes([17], 2, 2, 8)       # 2 pages: 1 candidate, budget clamps to 1
    assert small["step"] == 2 * (1 * 256 + (16 + 1) * 512 + 512) + 2 * 4 * 256 + 2 * 2 * 1 * 4


def test_header_is_plain_c_and_links_from_c(tmp_path):
    """include/kinetics_amd.h compiles as strict C99 and a C program linked against
    the library gets versions, sizes and argument errors without a GPU."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    exe = tmp_path / "use_from_c"
    libdir = _lib.LIB_PATH.parent
    subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", f"-I{HEADER.parent}",
                    str(ROOT / "tests" / "cabi" / "use_from_c.c"), "-o", str(exe), f"-L{libdir}", "-lkinetics_amd",
                    f"-Wl,-rpath,{libdir}"], check=True, capture_output=True, text=True)
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "ok" in run.stdout.splitlines()[-1]


def test_static_scratch_step_size_limit_is_checked_before_anything_else(lib):
    """The entry point that allocates nothing rejects shapes whose teams' scratch
    (shared keys and partial results) exceeds its built-in array, from the dimensions alone."""
    assert lib.kin_static_scratch_bytes() == 4 * 1024 * 1024 + 64 * 1024
    assert 0 < lib.kin_step_workspace_bytes(64, 1, 8192) <= lib.kin_static_scratch_bytes()
    assert lib.kin_step_workspace_bytes(64, 1, 16384) > lib.kin_static_scratch_bytes()
    st = lib.kin_blocktopk_decode_step_static(None, None, None, None, None, None, None, None, 128, 0, 1, None, None, None,
                                              None, 64, 4, 1, 128, 16, 1 << 20, 16384, 0, 0, 0.0, None, 0, None, None)
    assert st == _lib.KIN_ERR_WORKSPACE
    assert b"kin_blocktopk_decode_step_static" in lib.kin_last_error()
    # a shape that does not split needs no scratch: ordinary argument checking applies
    st = lib.kin_blocktopk_decode_step_static(None, None, None, None, None, None, None, None, 128, 0, 1, None, None, None,
                                              None, 4096, 4, 1, 128, 16, 1 << 20, 2048, 0, 0, 0.0, None, 0, None, None)
    assert st == _lib.KIN_ERR_NULL_POINTER
