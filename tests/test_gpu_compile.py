"""The ``kinetics::*`` operators under real compilation.

The reference wraps its kernels as ``mylib::*`` custom ops with fake kernels so that
the layer compiles with ``torch.compile(mode="max-autotune", fullgraph=True)``
(benchmark/blocktopk.py:41-43, benchmark/blocktopk_decoder.py:23-58,171-184).
Tracing alone (backend "eager") does not exercise what decides whether that is
correct: the schemas' mutation annotations, which AOT functionalisation uses to
keep an in-place cache append in the graph and in order.  Here every op goes
through ``torch.library.opcheck`` (schema, fake kernel, aliasing and mutation
under AOT dispatch), and functions built on them -- the three launches, the
fused step, the whole decoder layer -- are compiled with ``backend="aot_eager"``
and must leave the cache bytes, page lists and outputs of eager mode on two
consecutive steps with different k / v (an append that is dropped, duplicated or
reordered shows in the bytes).
"""
from types import SimpleNamespace

import pytest
import torch

from tests import problems as P

pytestmark = pytest.mark.gpu

D, PS = P.HEAD_DIM, P.PAGE_SIZE
DEV = "cuda"


@pytest.fixture(scope="module")
def ops():
    from kinetics_amd import ops as _ops

    return _ops


class State:
    """Device tensors of one small problem (fresh copies of its cache)."""

    def __init__(self, pb, ops, topk_cap=None):
        self.pb = pb
        self.q, self.k, self.v = (P.to_torch(x, DEV) for x in (pb.q, pb.k, pb.v))
        self.kv, self.kbar = P.to_torch(pb.kv_cache, DEV), P.to_torch(pb.kbar, DEV)
        self.idx, self.ptr, self.last = (P.int_tensor(x, DEV) for x in (pb.page_indices, pb.page_indptr, pb.last_page_len))
        cap = topk_cap or pb.topk + 1
        self.sel = torch.full((pb.B, pb.Hkv, cap), -7, dtype=torch.int32, device=DEV)
        self.cnt = torch.full((pb.B, pb.Hkv), -7, dtype=torch.int32, device=DEV)
        self.ws = torch.empty(max(16, ops.decode_workspace_bytes(pb.B, pb.Hq, pb.Hkv, cap, 3)), dtype=torch.uint8, device=DEV)
        self.step_ws = torch.empty(max(16, ops.step_workspace_bytes(pb.B, pb.Hkv, pb.kbar.shape[2])), dtype=torch.uint8, device=DEV)


def small_problem(seed=0):
    return P.make_problem(4200 + seed, [PS * 30 + 3, PS * 9, 1, PS * 17 + 16, PS * 50 + 7, PS * 12], num_kv_heads=2, group=4, topk=6)


def test_opcheck_every_operator(ops):
    """Schema against behaviour (which arguments are written), fake kernel against the real output,
    and the op under AOT dispatch with static and dynamic shapes, for every kinetics:: operator."""
    from torch.library import opcheck

    pb = small_problem()
    s = State(pb, ops)
    K = torch.ops.kinetics
    slots = torch.arange(pb.B, dtype=torch.int32, device=DEV)
    checks = [
        (K.append_paged_kv, (s.k, s.v, s.kv.clone(), s.kbar.clone(), s.idx, s.ptr, s.last), {}),
        (K.append_paged_kv, (s.k, s.v, s.kv.clone(), None, s.idx, s.ptr, s.last), {}),
        (K.append_paged_kv, (s.k, s.v, s.kv.clone(), s.kbar.clone(), s.idx, s.ptr, s.last, slots), {}),
        (K.update_kv, (s.k, s.v, torch.arange(pb.B + 1, dtype=torch.int32, device=DEV), s.kv.clone(), s.idx, s.ptr, s.last,
                       s.kbar.clone()), {}),
        (K.block_score_topk, (s.q, s.kbar, s.idx, s.ptr, s.last, pb.topk, s.sel.clone(), s.cnt.clone()), {}),
        (K.block_score_topk, (s.q, s.kbar, s.idx, s.ptr, s.last, pb.topk, s.sel.clone(), s.cnt.clone(), 0, 1, s.step_ws.clone(), PS,
                              slots), {}),
        (K.blocktopk_decode_step, (s.q, s.k, s.v, s.kv.clone(), s.kbar.clone(), s.idx, s.ptr, s.last, pb.topk, s.sel.clone(),
                                   s.cnt.clone(), 0.0), {}),
        (K.blocktopk_decode_step, (s.q, s.k, s.v, s.kv.clone(), s.kbar.clone(), s.idx, s.ptr, s.last, pb.topk, None, None, 0.0, 0, 1,
                                   0, s.step_ws.clone(), slots), {}),
    ]
    # the decode ops want a selection that exists
    ops.block_score_topk(s.q, s.kbar, s.idx, s.ptr, s.last, pb.topk, s.sel, s.cnt)
    checks += [
        (K.sparse_paged_decode, (s.q, s.kv, s.sel, s.cnt, s.last, None, 0.0, 1), {}),
        (K.sparse_paged_decode, (s.q, s.kv, s.sel, s.cnt, s.last, s.ws.clone(), 0.0, 3), {}),
        (K.dense_paged_decode, (s.q, s.kv, s.idx, s.ptr, s.last, pb.max_pages, None, 0.0, 1), {}),
        (K.dense_paged_decode, (s.q, s.kv, s.idx, s.ptr, s.last, pb.max_pages, s.ws.clone(), 0.0, 2), {}),
        (K.token_topk_decode, (s.q, s.kv, s.idx, s.ptr, s.last, 40, pb.max_pages, 4, 16, 0,
                               torch.empty(max(16, ops.token_topk_workspace_bytes(pb.B, pb.Hkv, pb.max_pages)), dtype=torch.uint8,
                                           device=DEV), 0.0), {}),
    ]
    # the row-wise layer ops
    x = torch.randn(6, 512, device=DEV).bfloat16()
    w = torch.randn(512, device=DEV).bfloat16()
    w128 = torch.randn(128, device=DEV).bfloat16()
    qkv = torch.randn(6, (4 + 2) * 128, device=DEV).bfloat16()
    checks += [
        (K.layer_norm, (x, 1e-6, w), {}),
        (K.qk_norm, (x.view(6, 4, 128), 1e-6, w128), {}),
        (K.fused_layer_norm, (x, x.clone(), 1e-6, w), {}),
        (K.qkv_norm_split, (qkv, w128, w128, 1e-6, 4, 1), {}),
        (K.gated_act, (x, x.flip(0).contiguous(), "silu"), {}),
    ]
    for op, args, kwargs in checks:
        opcheck(op, args, kwargs)


def _two_steps(fn, s):
    """fn(state, q, k, v) for two consecutive decode steps with different inputs; returns everything
    observable after each.  Between the steps every sequence grows by one token inside its open
    page (a host-side change of the table, outside the compiled function)."""
    gen = torch.Generator(device=DEV).manual_seed(99)
    res = []
    for step in range(2):
        q = torch.randn(s.q.shape, generator=gen, device=DEV).bfloat16()
        k = torch.randn(s.k.shape, generator=gen, device=DEV).bfloat16()
        v = torch.randn(s.v.shape, generator=gen, device=DEV).bfloat16()
        out = fn(s, q, k, v)
        torch.cuda.synchronize()
        res.append((out.clone(), s.kv.clone(), s.kbar.clone(), s.sel.clone(), s.cnt.clone()))
        if step == 0:
            assert int(s.last.max()) < PS
            s.last += 1
    return res


@pytest.mark.parametrize("path", ["three", "fused"])
def test_functions_on_the_ops_compile_with_aot_eager(ops, path):
    """backend="aot_eager", fullgraph=True: Dynamo traces, AOT autograd functionalises -- the
    in-place appends and the in-place page lists have to survive that, in order."""
    # sequences whose open page has room for a second token (the table itself is not rebuilt between the
    # two steps); one of them fills its page with the second token, which writes a mean key
    pb = P.make_problem(4300, [PS * 30 + 3, PS * 9 + 1, 2, PS * 17 + 15, PS * 50 + 7, PS * 12 + 5], num_kv_heads=2, group=4, topk=6)
    K = torch.ops.kinetics

    # the state's tensors are arguments, hence graph inputs whose mutation functionalisation has to keep
    def three(q, k, v, kv, kbar, idx, ptr, last, sel, cnt, ws, step_ws):
        K.append_paged_kv(k, v, kv, kbar, idx, ptr, last)
        K.block_score_topk(q, kbar, idx, ptr, last, pb.topk, sel, cnt)
        o = K.sparse_paged_decode(q, kv, sel, cnt, last, ws, 0.0, 3)
        return o + 0.0

    def fused(q, k, v, kv, kbar, idx, ptr, last, sel, cnt, ws, step_ws):
        o = K.blocktopk_decode_step(q, k, v, kv, kbar, idx, ptr, last, pb.topk, sel, cnt, 0.0, 0, 1, 0, step_ws)
        return o + 0.0

    body = three if path == "three" else fused
    torch._dynamo.reset()
    compiled = torch.compile(body, backend="aot_eager", fullgraph=True)

    def on_state(fn):
        return lambda s, q, k, v: fn(q, k, v, s.kv, s.kbar, s.idx, s.ptr, s.last, s.sel, s.cnt, s.ws, s.step_ws)

    eager = _two_steps(on_state(body), State(pb, ops))
    got = _two_steps(on_state(compiled), State(pb, ops))
    for step, (e, g) in enumerate(zip(eager, got)):
        names = ("output", "kv_cache", "kbar", "page lists", "list lengths")
        for name, a, b in zip(names, e, g):
            assert torch.equal(a, b), f"step {step}: {name} differs between eager and aot_eager"
    # the two steps did append two different rows (the comparison above would not see a no-op)
    assert not torch.equal(eager[0][1], eager[1][1])
    assert not torch.equal(eager[0][2], eager[1][2])  # and the page that filled got its mean key


@pytest.mark.timeout(400)
@pytest.mark.parametrize("fused", [True, False], ids=["one-launch", "three-launches"])
@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_decoder_layer_compiles(ops, backend, fused):
    """BlockTopkDecoderLayer.forward compiled as the reference compiles its layer (fullgraph=True):
    two consecutive steps leave the cache bytes, page lists and outputs of the eager layer."""
    from kinetics_amd.decoder_layer import BlockTopkDecoderLayer, init_weights

    cfg = SimpleNamespace(num_attention_heads=8, num_key_value_heads=2, head_dim=D, hidden_size=512, intermediate_size=1024,
                          rms_norm_eps=1e-6, hidden_act="silu")
    B, prefix, topk = 6, PS * 40, 8

    def make():
        torch.manual_seed(11)
        layer = BlockTopkDecoderLayer(cfg, 2, B, prefix, prefix + 512, PS, topk, DEV, torch.bfloat16, seed=5)
        layer.apply(init_weights)
        layer.eval().to(DEV, dtype=torch.bfloat16)
        layer.prepare_wrapper(prefix)
        layer.attn.fused = fused
        return layer

    hs = [torch.randn(B, 1, 512, generator=torch.Generator().manual_seed(i)).bfloat16().to(DEV) for i in range(2)]

    def run(layer, fwd):
        res = []
        for h in hs:
            out = fwd(h.clone())
            torch.cuda.synchronize()
            a = layer.attn
            res.append((out.clone(), a.kv_cache.clone(), a.compressed_key_cache.clone(), a.topk_page_indices.clone(),
                        a.topk_page_count.clone()))
        return res

    if backend == "inductor":
        import torch._inductor.config as inductor_config

        inductor_config.compile_threads = 1  # no pool of compile workers beside the GPU process
    torch._dynamo.reset()  # many layers are compiled in one test process: each starts with an empty code cache
    ref_layer = make()
    eager = run(ref_layer, ref_layer.forward)
    layer = make()
    try:
        compiled = torch.compile(layer.forward, backend=backend, fullgraph=True)
        got = run(layer, compiled)
    except Exception as e:  # noqa: BLE001 -- a code generator that cannot run on this machine is not this library's failure
        if backend == "inductor":
            pytest.skip(f"Inductor does not run here: {type(e).__name__}: {str(e)[:200]}")
        raise
    for step, (e, g) in enumerate(zip(eager, got)):
        names = ("output", "kv_cache", "compressed_key_cache", "page lists", "list lengths")
        for name, a, b in zip(names, e, g):
            if name == "output" and backend == "inductor":
                # generated elementwise code may round an intermediate differently from the eager kernels
                assert torch.allclose(a.float(), b.float(), rtol=3e-2, atol=3e-2), f"step {step}: {name}"
            else:
                assert torch.equal(a, b), f"step {step}: {name} differs between eager and {backend}"
