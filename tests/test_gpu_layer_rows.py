"""The row-wise layer kernels (RMSNorm with the residual add, q/k norm + split,
gated activation) through the C ABI against the oracle.

Bar: outputs within one unit in the last place of the oracle's float64 result
(the kernels keep fp32 statistics; two units for the float16 gated product, whose
rounded activation can fall on either side of a float16 boundary), which is inside the 2e-2 tolerance of the
attention path; the updated residual, a single rounded add, is bit-exact, and so
are copied v heads.  Every case runs for bfloat16 and for float16 tensors (the
kin_*_f16 entry points)."""
import numpy as np
import pytest
import torch

from oracle import blocktopk_oracle as O
from tests import problems as P

pytestmark = pytest.mark.gpu
DEV = "cuda"
D = P.HEAD_DIM


@pytest.fixture(scope="module")
def ops():
    from kinetics_amd import ops as _ops

    return _ops


@pytest.fixture(params=["bf16", "f16"], autouse=True)
def fmt(request):
    """Every test of this file runs once per element format."""
    with O.element_format(request.param):
        yield request.param


def rand_bits(rng, shape, scale=1.0):
    return O.f32_to_elem(rng.standard_normal(shape).astype(np.float32) * scale)


def ulps(a_bits, b_bits):
    def key(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, 0x8000 - b, b)

    near = np.abs(O.elem_to_f32(a_bits).astype(np.float64) - O.elem_to_f32(b_bits)) <= 1e-6
    return int(np.where(near, 0, np.abs(key(a_bits) - key(b_bits))).max())


def check_close(got_bits, want_bits, max_ulps=1):
    assert got_bits.shape == want_bits.shape
    assert ulps(got_bits, want_bits) <= max_ulps
    g, w = O.elem_to_f32(got_bits), O.elem_to_f32(want_bits)
    assert np.allclose(g, w, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("rows,hidden", [(1, 128), (37, 128), (1, 64), (777, 64), (16, 256), (6, 896), (33, 2048), (5, 1024), (9, 5120),
                                         (3, 8192), (1027, 4096), (4, 512)])
@pytest.mark.parametrize("residual", [False, True])
def test_rms_norm(ops, rows, hidden, residual):
    rng = np.random.default_rng(rows * 7 + hidden)
    x = rand_bits(rng, (rows, hidden), 2.0)
    w = O.f32_to_elem(1 + 0.3 * rng.standard_normal(hidden).astype(np.float32))
    r = rand_bits(rng, (rows, hidden), 3.0) if residual else None
    want, want_r = O.rms_norm(x, w, 1e-6, residual=r)
    xt, wt = P.to_torch(x, DEV), P.to_torch(w, DEV)
    rt = P.to_torch(r, DEV) if residual else None
    out = ops.rms_norm(xt, wt, 1e-6, residual=rt)
    torch.cuda.synchronize()
    assert np.array_equal(P.from_torch(xt), x)  # the input is left alone
    check_close(P.from_torch(out), want)
    if residual:
        assert np.array_equal(P.from_torch(rt), want_r)


def test_rms_norm_strided_rows_and_in_place(ops):
    rng = np.random.default_rng(3)
    wide = rand_bits(rng, (19, 3 * 512), 1.5)
    w = O.f32_to_elem(1 + 0.2 * rng.standard_normal(512).astype(np.float32))
    wide_t, wt = P.to_torch(wide, DEV), P.to_torch(w, DEV)
    want, _ = O.rms_norm(wide[:, 512:1024], w, 1e-5)
    out_wide = torch.zeros(19, 1024, dtype=wide_t.dtype, device=DEV)
    got = ops.rms_norm(wide_t[:, 512:1024], wt, 1e-5, out=out_wide[:, 512:])
    torch.cuda.synchronize()
    check_close(P.from_torch(got), want)
    assert torch.count_nonzero(out_wide[:, :512]).item() == 0  # nothing written outside the view
    # out aliasing x, as flashinfer's fused form updates hidden_states in place
    ops.rms_norm(wide_t[:, 512:1024], wt, 1e-5, out=wide_t[:, 512:1024])
    torch.cuda.synchronize()
    after = P.from_torch(wide_t)
    check_close(after[:, 512:1024], want)
    assert np.array_equal(after[:, :512], wide[:, :512]) and np.array_equal(after[:, 1024:], wide[:, 1024:])
    # 4-D rows as qk_norm takes them (benchmark/model_utils.py:15-25)
    q = rand_bits(rng, (3, 1, 4, D))
    wq = O.f32_to_elem(1 + 0.2 * rng.standard_normal(D).astype(np.float32))
    got_q = torch.ops.kinetics.qk_norm(P.to_torch(q, DEV), 1e-6, P.to_torch(wq, DEV))
    assert got_q.shape == (3, 1, 4, D)
    check_close(P.from_torch(got_q), O.rms_norm(q, wq, 1e-6)[0])


def test_norm_ops_by_the_reference_names(ops):
    rng = np.random.default_rng(4)
    h = rand_bits(rng, (5, 1, 1024))
    r = rand_bits(rng, (5, 1, 1024))
    w = O.f32_to_elem(1 + 0.2 * rng.standard_normal(1024).astype(np.float32))
    ht, rt, wt = P.to_torch(h, DEV), P.to_torch(r, DEV), P.to_torch(w, DEV)
    out = torch.ops.kinetics.layer_norm(ht, 1e-6, wt)
    assert out.shape == (5, 1, 1024)
    check_close(P.from_torch(out), O.rms_norm(h, w, 1e-6)[0])
    want, want_r = O.rms_norm(h, w, 1e-6, residual=r)
    out2 = torch.ops.kinetics.fused_layer_norm(ht, rt, 1e-6, wt)
    torch.cuda.synchronize()
    check_close(P.from_torch(out2), want)
    assert np.array_equal(P.from_torch(rt), want_r)
    with pytest.raises(ValueError):
        ops.rms_norm(ht, wt[:512], 1e-6)
    with pytest.raises(ValueError, match="KIN_ERR_UNSUPPORTED"):
        ops.rms_norm(ht[..., :1000].contiguous(), wt[:1000].contiguous(), 1e-6)


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("B,Hq,Hkv,pad", [(7, 4, 1, 0), (130, 8, 8, 0), (1, 5, 1, 0), (33, 8, 2, 64), (4096, 4, 1, 0)])
def test_qkv_norm_split(ops, B, Hq, Hkv, pad, D):
    rng = np.random.default_rng(B + Hq)
    width = (Hq + 2 * Hkv) * D
    buf = rand_bits(rng, (B, width + pad), 2.0)
    qw = O.f32_to_elem(1 + 0.3 * rng.standard_normal(D).astype(np.float32))
    kw = O.f32_to_elem(1 + 0.3 * rng.standard_normal(D).astype(np.float32))
    wq, wk, wv = O.qkv_norm_split(buf[:, :width], qw, kw, 1e-6, Hq, Hkv, head_dim=D)
    bt = P.to_torch(buf, DEV)
    q, k, v = ops.qkv_norm_split(bt[:, :width], P.to_torch(qw, DEV), P.to_torch(kw, DEV), 1e-6, Hq, Hkv)
    torch.cuda.synchronize()
    assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
    check_close(P.from_torch(q), wq)
    check_close(P.from_torch(k), wk)
    assert np.array_equal(P.from_torch(v), wv)
    assert np.array_equal(P.from_torch(bt), buf)


@pytest.mark.parametrize("act", ["silu", "gelu", "relu"])
@pytest.mark.parametrize("rows,inter", [(1, 8), (5, 1536), (257, 3072), (3, 25600)])
def test_gated_act(ops, act, rows, inter):
    rng = np.random.default_rng(rows + inter)
    fused = rand_bits(rng, (rows, 2 * inter), 3.0)
    want = O.gated_act(fused[:, :inter], fused[:, inter:], act)
    ft = P.to_torch(fused, DEV)
    # the two halves of one fused projection
    got = ops.gated_act(ft[:, :inter], ft[:, inter:], act)
    # and two separate contiguous tensors
    got2 = ops.gated_act(ft[:, :inter].contiguous(), ft[:, inter:].contiguous(), act)
    torch.cuda.synchronize()
    # float16 keeps 11 bits: an fp32-rounding difference in act(gate) now and then lands on the other side of a
    # float16 boundary, and the product then differs by up to two units
    check_close(P.from_torch(got), want, max_ulps=2 if got.dtype == torch.float16 else 1)
    assert torch.equal(got, got2)
    assert np.array_equal(P.from_torch(ft), fused)


def test_row_kernels_accept_empty_batches(ops, fmt):
    dt = torch.float16 if fmt == "f16" else torch.bfloat16
    other = torch.bfloat16 if fmt == "f16" else torch.float16
    w = torch.ones(512, dtype=dt, device=DEV)
    assert ops.rms_norm(torch.empty(0, 512, dtype=dt, device=DEV), w, 1e-6).shape == (0, 512)
    e = torch.empty(0, 64, dtype=dt, device=DEV)
    assert ops.gated_act(e, e).shape == (0, 64)
    q, k, v = ops.qkv_norm_split(torch.empty(0, 6 * D, dtype=dt, device=DEV), w[:D].contiguous(),
                                 w[:D].contiguous(), 1e-6, 4, 1)
    assert q.shape == (0, 4, D) and k.shape == (0, 1, D) and v.shape == (0, 1, D) and q.dtype == dt
    with pytest.raises(ValueError):
        ops.gated_act(torch.zeros(2, 64, dtype=dt, device=DEV), e)
    with pytest.raises(ValueError):
        ops.gated_act(e, e, act="tanh")
    # one format per call: mixed tensors are refused, so is fp32
    with pytest.raises(TypeError):
        ops.rms_norm(torch.zeros(2, 512, dtype=dt, device=DEV), w.to(other), 1e-6)
    with pytest.raises(TypeError):
        ops.gated_act(torch.zeros(2, 64, dtype=dt, device=DEV), torch.zeros(2, 64, dtype=other, device=DEV))
    with pytest.raises(TypeError):
        ops.rms_norm(torch.zeros(2, 512, dtype=torch.float32, device=DEV), w, 1e-6)
