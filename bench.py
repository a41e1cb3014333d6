#!/usr/bin/env python3
"""Throughput of one block top-k sparse decode step on one MI355X.

A "step" is what benchmark/blocktopk_decoder.py:209-225 does for one batch:
append the new token's K/V, score every page against the group-mean query,
take the top-k pages plus the last page, attend over them.  The harness mirrors
benchmark/blocktopk.py:47-61: W untimed warm-up steps, then K timed steps
between device synchronisations, throughput = K * batch / elapsed (tokens/s for
one layer on one GPU's share of the heads).  Sequence lengths stay fixed across
steps, as in the reference harness whose metadata never changes.

Prints ONE JSON line.  ``value`` is decode tokens/s per layer with every input
already resident in HBM.  ``roofline`` describes the dominant kernel (the fused
step kernel, or the sparse paged attention with --mode three); its ``achieved``
is algorithmic bytes over the kernel's HIP-event time measured in this run,
while ``traffic`` is NOT measured by this run: it is read from
profiles/hbm_traffic.json, which holds the rocprofv3 --pmc FETCH_SIZE /
WRITE_SIZE figures of an earlier run of the same kernel and workload
(``traffic_source`` says so in the line).  ``step_hbm`` is the whole step
against the algorithmic-bytes model, ``cpu_baseline`` the torch-CPU restatement
of the reference path timed on this machine's host cores (a slice of the
headline workload, and the tiny configuration in full), ``dense_baseline`` the
dense paged decode on the same tensors.  For the headline workload the same
line also carries ``workloads`` (the other BASELINE configurations, each
measured the same way on its own cache), ``token_topk`` / ``strided_topk``
(LiteSys' token-granular policies on the headline cache) and the figure in the
reference's printed normalisation (divided by world_size * num_hidden_layers,
benchmark/blocktopk.py:82).
"""
from __future__ import annotations

import argparse
import contextlib
import gc
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
PS, D = 16, 128

WORKLOADS = {
    # name: (batch, ctx, H_kv, group, topk, description)
    "qwen3-8b-share": (4096, 32768, 1, 4, 128, "Qwen3-8B one-GPU share (TP=8): 1 KV head, 4 Q heads"),
    "qwen3-32b-share": (1024, 32768, 1, 8, 256, "Qwen3-32B one-GPU share: 1 KV head, 8 Q heads"),
    "qwen3-8b-tp1": (512, 32768, 8, 4, 128, "Qwen3-8B unsharded attention: 8 KV heads, 32 Q heads"),
    "tiny": (8, 4096, 1, 4, 64, "CPU-runnable tiny case"),
    # the command in the reference's benchmark/README.md: --batch_size 256 --gen_len 32768 (ctx 16384) --topk_page 64
    "qwen3-8b-readme": (256, 16384, 1, 4, 64, "reference README example: Qwen3-8B share, B=256, ctx 16K, 64 pages"),
    # ragged: contexts uniform in [1024, ctx], budget min(topk, pages), half the tables fragmented
    "qwen3-0.6b-mix": (512, 32768, 8, 2, 64, "continuous-batching mix, Qwen3-0.6B attention: 8 KV heads, 16 Q heads"),
}
RAGGED = {"qwen3-0.6b-mix"}


def algorithmic_bytes(lengths, Hkv, G, topk, PS=PS):
    """Bytes per step that the algorithm has to move (bf16 K/V, int32 indices),
    summed over sequences with post-append token counts ``lengths``."""
    Hq = Hkv * G
    step = attn = score = dense = 0
    for L in lengths:
        n_pages = (L + PS - 1) // PS
        n_cand = n_pages - 1
        last_len = L - n_cand * PS
        k_eff = min(topk, n_cand)
        kbar = Hkv * n_cand * D * 2
        kv_sel = Hkv * (k_eff * PS + last_len) * 2 * D * 2
        append = Hkv * 2 * D * 2
        qo = 2 * Hq * D * 2
        step += kbar + kv_sel + append + qo + 2 * Hkv * k_eff * 4
        attn += kv_sel + qo + Hkv * (k_eff + 1) * 4
        score += kbar + Hq * D * 2 + Hkv * (k_eff + 1) * 4
        dense += Hkv * (L * 2 * D * 2 + append) + qo
    return dict(step=step, attention=attn, score_select=score, dense=dense, per_seq=step / max(1, len(lengths)))


def build_state(torch, ops, B, ctx, Hkv, G, topk, device, seed=2, ragged=False, kv_alloc=None, PS=PS, dtype=None):
    """Paged cache, K ~ N(0,1) + per-page mean offset N(0,0.5), V ~ N(0,1); kbar =
    true page means.  Uniform workloads use the reference layout (page id =
    p*B + b, max_len = ctx+512, every context ``ctx`` tokens + the appended one).
    Ragged ones draw contexts uniformly from [1024, ctx] (seed 3); even
    sequences own contiguous page runs, odd ones pages from a shuffled free list."""
    dtype = dtype or torch.bfloat16
    n_full = ctx // PS
    max_pages = (ctx + 512) // PS
    gen = torch.Generator(device=device).manual_seed(seed)
    if ragged:
        import numpy as np

        rng = np.random.default_rng(3)
        lengths = rng.integers(1024, ctx + 1, size=B) + 1
        n_pages = (lengths + PS - 1) // PS
        num_pages = int(n_pages.sum())
        indptr_np = np.zeros(B + 1, dtype=np.int64)
        indptr_np[1:] = np.cumsum(n_pages)
        ids = np.empty(num_pages, dtype=np.int64)
        even = [b for b in range(B) if b % 2 == 0]
        cur = 0
        for b in even:
            ids[indptr_np[b]:indptr_np[b + 1]] = np.arange(cur, cur + n_pages[b])
            cur += n_pages[b]
        rest = rng.permutation(np.arange(cur, num_pages))
        pos = 0
        for b in range(1, B, 2):
            ids[indptr_np[b]:indptr_np[b + 1]] = rest[pos:pos + n_pages[b]]
            pos += n_pages[b]
        last_np = (lengths - (n_pages - 1) * PS).astype(np.int32)
        max_pages = int(n_pages.max())
    else:
        num_pages = max_pages * B
        lengths = [ctx + 1] * B
    kv_shape = (num_pages, 2, PS, Hkv, D)
    kv = kv_alloc(kv_shape) if kv_alloc else torch.empty(kv_shape, dtype=dtype, device=device)
    chunk = max(1, (1 << 28) // (2 * PS * Hkv * D))
    for s in range(0, num_pages, chunk):
        e = min(num_pages, s + chunk)
        x = torch.randn(e - s, 2, PS, Hkv, D, generator=gen, device=device, dtype=torch.float32)
        mu = torch.randn(e - s, 1, 1, Hkv, 1, generator=gen, device=device, dtype=torch.float32) * 0.5
        x[:, 0:1] += mu
        kv[s:e] = x.to(dtype)
        del x, mu
    if ragged:
        indices = torch.from_numpy(ids.astype("int32")).to(device)
        indptr = torch.from_numpy(indptr_np.astype("int32")).to(device)
        last = torch.from_numpy(last_np).to(device)
    else:
        table = torch.arange(n_full + 1, dtype=torch.int32, device=device) * B + torch.arange(B, dtype=torch.int32, device=device)[:, None]
        indices = table.reshape(-1).contiguous()
        indptr = (torch.arange(B + 1, dtype=torch.int32, device=device) * (n_full + 1)).contiguous()
        last = torch.ones(B, dtype=torch.int32, device=device)
    st = dict(
        kv=kv,
        indices=indices,
        indptr=indptr,
        last=last,
        lengths=[int(x) for x in lengths],
        kbar=torch.zeros(B, Hkv, max_pages, D, dtype=dtype, device=device),
        sel=torch.full((B, Hkv, topk + 1), -1, dtype=torch.int32, device=device),
        cnt=torch.zeros(B, Hkv, dtype=torch.int32, device=device),
        q=torch.randn(B, Hkv * G, D, generator=gen, device=device, dtype=torch.float32).to(dtype),
        k=torch.randn(B, Hkv, D, generator=gen, device=device, dtype=torch.float32).to(dtype),
        v=torch.randn(B, Hkv, D, generator=gen, device=device, dtype=torch.float32).to(dtype),
        out=torch.empty(B, Hkv * G, D, dtype=dtype, device=device),
        n_full=n_full, max_pages=max_pages, num_pages=num_pages,
    )
    st["page_size"] = PS
    st["max_pages_used"] = max((L + PS - 1) // PS for L in st["lengths"])
    ops.build_kbar(st["kv"], st["kbar"], st["indices"], st["indptr"], st["last"])
    ws = ops.decode_workspace_bytes(B, Hkv * G, Hkv, topk + 1)
    st["ws"] = torch.empty(max(ws, 16), dtype=torch.uint8, device=device)
    wsd = ops.decode_workspace_bytes(B, Hkv * G, Hkv, st["max_pages_used"])
    st["ws_dense"] = torch.empty(max(wsd, 16), dtype=torch.uint8, device=device)
    return st


def cpu_baseline(torch, B_cpu, ctx, G, topk, budget_s=20.0):
    """The reference's torch path (oracle/torch_path.py) on the host cores, on a
    slice of the workload: B_cpu sequences of the same context length.  Scores in
    bf16 as the reference computes them (benchmark/blocktopk_decoder.py:216), and
    in fp32 beside it."""
    from oracle import torch_path

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    n_full = ctx // PS
    n_pages = n_full + 1
    g = torch.Generator().manual_seed(5)
    kv = torch.empty(B_cpu * n_pages, 2, PS, 1, D, dtype=torch.bfloat16)
    chunk = 1 << 13
    for s in range(0, kv.shape[0], chunk):
        e = min(kv.shape[0], s + chunk)
        kv[s:e] = torch.randn(e - s, 2, PS, 1, D, generator=g).to(torch.bfloat16)
    table = (torch.arange(n_pages)[None, :] * B_cpu + torch.arange(B_cpu)[:, None]).contiguous()
    kbar = kv[table[:, :-1], 0, :, 0].float().mean(dim=2).to(torch.bfloat16)  # [B, n_full, D]
    q = torch.randn(B_cpu, G, D, generator=g).to(torch.bfloat16)
    k = torch.randn(B_cpu, 1, D, generator=g).to(torch.bfloat16)
    v = torch.randn(B_cpu, 1, D, generator=g).to(torch.bfloat16)
    last = torch.ones(B_cpu, dtype=torch.int64)
    med, count = {}, {}
    for dt in (torch.bfloat16, torch.float32):
        times = []
        for _ in range(3):
            torch_path.blocktopk_decode_step(q, k, v, kv, kbar, table, last, topk, compute_dtype=dt)
        t_end = time.perf_counter() + budget_s / 2
        while len(times) < 5 or (time.perf_counter() < t_end and len(times) < 200):
            t0 = time.perf_counter()
            torch_path.blocktopk_decode_step(q, k, v, kv, kbar, table, last, topk, compute_dtype=dt)
            times.append(time.perf_counter() - t0)
        med[dt], count[dt] = statistics.median(times), len(times)
    m = med[torch.bfloat16]
    return dict(value=B_cpu / m, unit="tokens/s", cores=cores, cpu_model=cpu_model_name(), kind="port",
                value_fp32_scores=B_cpu / med[torch.float32],
                sample=f"torch-CPU restatement of the reference path (oracle/torch_path.py), {B_cpu} of the batch's "
                       f"sequences at ctx={ctx}, k={topk}, page scores in bf16 as the reference computes them "
                       f"(value_fp32_scores: in fp32), median of {count[torch.bfloat16]} steps after 3 warm-ups, "
                       f"{m * 1e3:.2f} ms/step; tokens/s is linear in batch")


# (world_size, num_hidden_layers) the reference's printed figure is divided by (benchmark/blocktopk.py:82)
REFERENCE_NORMALISATION = {"qwen3-8b-share": (8, 36), "qwen3-8b-readme": (8, 36), "qwen3-32b-share": (8, 64)}

WHOLE_LAYER_MODEL = {"qwen3-8b-share": ("Qwen3-8B", 8), "qwen3-32b-share": ("Qwen3-32B", 8),
                     "qwen3-8b-readme": ("Qwen3-8B", 8)}


def whole_layer(torch, args, B, ctx, topk, device):
    """One whole decoder layer of the TP shard, timed like benchmark/blocktopk.py:47-61
    (hidden_states.clone() -> forward, warm-up then K timed calls).  The printed figure
    of the reference additionally divides by world_size * num_hidden_layers (:82)."""
    from kinetics_amd.decoder_layer import BlockTopkDecoderLayer, init_weights, qwen3_config

    name, world = WHOLE_LAYER_MODEL[args.workload]
    cfg = qwen3_config(name)
    elem = torch.float16 if args.dtype == "float16" else torch.bfloat16   # the whole layer moves to --dtype, as in the reference
    layer = BlockTopkDecoderLayer(cfg, world, B, ctx, ctx + 512, PS, topk, device, elem)
    layer.apply(init_weights)
    layer.eval().to(device, dtype=elem)
    hidden = torch.randn(B, 1, cfg.hidden_size, device=device, dtype=elem)
    for _ in range(args.warmup):
        layer(hidden.clone())
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        layer(hidden.clone())
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    # the same forward replayed as one HIP graph (the reference compiles its layer
    # with mode="max-autotune", benchmark/blocktopk.py:41-43)
    graphed = layer.graphed(hidden)
    for _ in range(args.warmup):
        graphed(hidden)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        graphed(hidden)
    torch.cuda.synchronize()
    dt_graph = (time.perf_counter() - t0) / args.steps
    del graphed
    out = {"model": name, "world_size": world, "ms_per_layer_step": dt * 1e3, "tokens_per_s_per_layer": B / dt,
           "ms_per_layer_step_hip_graph": dt_graph * 1e3, "tokens_per_s_per_layer_hip_graph": B / dt_graph,
           "normalised_like_reference_print": B / dt / (world * cfg.num_hidden_layers),
           "note": "GEMMs are hipBLASLt through PyTorch; norms, q/k/v split, attention and the gated activation are this repository's kernels"}
    del layer
    torch.cuda.empty_cache()
    if not args.no_dense:
        # the reference's dense layer (benchmark/dense.py, dense_decoder.py) on the same shape
        from kinetics_amd.decoder_layer import DenseDecoderLayer

        dense = DenseDecoderLayer(cfg, world, B, ctx, ctx + 512, PS, device, elem)
        dense.apply(init_weights)
        dense.eval().to(device, dtype=elem)
        dense.prepare_wrapper()
        nd = max(3, min(args.steps, 20))
        for _ in range(2):
            dense(hidden.clone())
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(nd):
            dense(hidden.clone())
        torch.cuda.synchronize()
        dd = (time.perf_counter() - t0) / nd
        out["dense_layer"] = {"ms_per_layer_step": dd * 1e3, "tokens_per_s_per_layer": B / dd, "steps": nd,
                              "normalised_like_reference_print": B / dd / (world * cfg.num_hidden_layers)}
        out["sparse_over_dense_layer"] = dd / dt
        del dense
        torch.cuda.empty_cache()
    return out


def cpu_model_name():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


LAST_LAUNCH_MS = []
LAST_GRAPH_REPLAY_MS = None
LAST_GRAPH_REPLAY_10_MS = None   # ten steps per graph


@contextlib.contextmanager
def collector_paused():
    """A timed loop without the interpreter's cyclic collector (as timeit does): a
    full collection that lands between two launches stalls the host for tens of
    milliseconds, and the GPU idles through it inside the timed K steps."""
    was = gc.isenabled()
    gc.collect()
    gc.disable()
    try:
        yield
    finally:
        if was:
            gc.enable()


GRAPH_REPLAY_BELOW_MS = 0.1   # steps shorter than this are host-bound when launched eagerly


def time_graph_replay(torch, step, steps, warmup, per_graph=1):
    """The step captured as a HIP graph and replayed: what the GPU does when
    the host is out of the way (the launch-overhead half of the reference's
    torch.compile(mode="max-autotune"), benchmark/blocktopk.py:41-43).  The graph holds
    ``per_graph`` consecutive steps (a served model replays one graph per forward pass,
    a step per layer: each replay costs a few microseconds of its own, which one step per
    graph pays in full); about ``steps`` steps in all are queued back to back between
    two synchronisations; ms per step."""
    cur = torch.cuda.current_stream()
    side = torch.cuda.Stream()
    side.wait_stream(cur)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        step()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(per_graph):
                step()
    cur.wait_stream(side)
    torch.cuda.synchronize()
    replays = max(1, steps // per_graph)
    with collector_paused():
        for _ in range(max(1, warmup // per_graph)):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(replays):
            graph.replay()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / (replays * per_graph)
    del graph
    return dt * 1e3


def time_step(torch, ops, st, B, Hkv, topk, steps, warmup, mode="auto"):
    """W untimed and K timed decode steps on the state ``st``, timed by the host clock between two
    synchronisations and by HIP events on the launch stream: one pair around the timed region when
    the step is one call (the fused step), a record between all launches when it is three.  Returns
    (ms_per_step, elapsed_s, {kernel: mean ms}, fused?).  When the eager step is shorter than
    GRAPH_REPLAY_BELOW_MS, LAST_GRAPH_REPLAY_MS also holds the same step replayed
    as a HIP graph (None otherwise)."""
    device = st["q"].device
    fused = mode == "fused" or (mode == "auto" and ops.prefer_fused_step(B, Hkv, st["max_pages_used"], topk))
    # few long lists: the scoring of a list is shared by several workgroups that meet through this
    sws = ops.step_workspace_bytes(B, Hkv, st["kbar"].shape[2])
    step_ws = torch.empty(sws, dtype=torch.uint8, device=device) if sws else None
    if fused:
        kernels = [("fused_step", lambda: ops.blocktopk_decode_step(
            st["q"], st["k"], st["v"], st["kv"], st["kbar"], st["indices"], st["indptr"], st["last"], topk,
            out=st["out"], workspace=step_ws))]
    else:
        kernels = [
            ("append", lambda: ops.append_paged_kv(st["k"], st["v"], st["kv"], st["kbar"], st["indices"], st["indptr"],
                                                   st["last"])),
            ("score_topk", lambda: ops.block_score_topk(st["q"], st["kbar"], st["indices"], st["indptr"], st["last"], topk,
                                                        st["sel"], st["cnt"], workspace=step_ws, page_size=st["page_size"])),
            ("sparse_attention", lambda: ops.sparse_paged_decode(st["q"], st["kv"], st["sel"], st["cnt"], st["last"],
                                                                 out=st["out"], workspace=st["ws"])),
        ]
    K = steps
    # Events on the launch stream.  A step that is one kernel gets one pair around the K launches of the
    # timed region: its average launch duration is their distance / K (the ~1 us between dependent
    # launches included).  An event record is a packet of its own in the queue and holds the next kernel
    # back by 2.5-5 us (qwen3-8b-readme: 38.6-40.6 us per step with no record between the launches, 41.2
    # with one, 46.6 with two), so records between the launches would time themselves; the reference's
    # loop has none either (benchmark/blocktopk.py:47-61).  A step of several kernels needs the records
    # between them to tell the kernels apart, and pays for them.
    per_launch = len(kernels) > 1
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(len(kernels) + 1)] for _ in range(K if per_launch else 0)]
    region = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
    # the collection happens before the warm-up, so that nothing but a synchronise lies between the
    # warm-up and the timed steps (a GPU left idle for the tens of milliseconds of a collection runs
    # its next launches slower: 1.5 % on 20 timed steps)
    with collector_paused():
        for _ in range(warmup):
            for _, fn in kernels:
                fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        region[0].record()
        if per_launch:
            for i in range(K):
                ev[i][0].record()
                for j, (_, fn) in enumerate(kernels):
                    fn()
                    ev[i][j + 1].record()
        else:
            fn = kernels[0][1]
            for _ in range(K):
                fn()
        region[1].record()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        # after the timed region: a few launches bracketed one by one, for the spread between launches
        P = K if per_launch else min(K, 20)
        if not per_launch:
            ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(P)]
            for i in range(P):
                ev[i][0].record()
                fn()
                ev[i][1].record()
            torch.cuda.synchronize()
    global LAST_LAUNCH_MS, LAST_GRAPH_REPLAY_MS, LAST_GRAPH_REPLAY_10_MS
    LAST_LAUNCH_MS = [round(sum(e[j].elapsed_time(e[j + 1]) for j in range(len(kernels))), 3) for e in ev]
    if per_launch:
        kernel_ms = {name: statistics.fmean(e[j].elapsed_time(e[j + 1]) for e in ev) for j, (name, _) in enumerate(kernels)}
    else:
        kernel_ms = {kernels[0][0]: region[0].elapsed_time(region[1]) / K}
    LAST_GRAPH_REPLAY_MS = LAST_GRAPH_REPLAY_10_MS = None
    if elapsed / K * 1e3 < GRAPH_REPLAY_BELOW_MS:
        def whole_step():
            for _, fn in kernels:
                fn()
        LAST_GRAPH_REPLAY_MS = time_graph_replay(torch, whole_step, K, warmup)
        LAST_GRAPH_REPLAY_10_MS = time_graph_replay(torch, whole_step, K, warmup, per_graph=10)
    return elapsed / K * 1e3, elapsed, kernel_ms, fused


def time_dense(torch, ops, st, nd):
    """The dense baseline (benchmark/dense_decoder.py:211-219) on the same tensors: ms per step."""
    with collector_paused():
        for _ in range(2):
            ops.dense_paged_decode(st["q"], st["kv"], st["indices"], st["indptr"], st["last"], st["max_pages_used"],
                                   out=st["out"], workspace=st["ws_dense"])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(nd):
            ops.append_paged_kv(st["k"], st["v"], st["kv"], None, st["indices"], st["indptr"], st["last"])
            ops.dense_paged_decode(st["q"], st["kv"], st["indices"], st["indptr"], st["last"], st["max_pages_used"],
                                   out=st["out"], workspace=st["ws_dense"])
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / nd * 1e3


def time_token_policies(torch, ops, st, B, Hkv, G, topk, nt, traffic_of):
    """LiteSys' token-granular policies on the same cache with the same token
    budget (topk_pages * 16 tokens, 4 sink tokens, a 16-token window): every key of
    the context is streamed once (256 B per token), then the listed tokens' K and V rows."""
    device = st["q"].device
    ntok, sink, window = topk * PS, 4, 16
    res = {}
    row = 2 * D   # bytes of one head row
    tok_bytes = sum(Hkv * (L * row + min(L, ntok + sink + window) * 2 * row + 2 * row) + 2 * Hkv * G * row for L in st["lengths"])
    ws_tok = torch.empty(max(16, ops.token_topk_workspace_bytes(B, Hkv, st["max_pages_used"])), dtype=torch.uint8, device=device)
    ws_str = torch.empty(max(16, ops.strided_topk_workspace_bytes(B, Hkv, st["max_pages_used"])), dtype=torch.uint8, device=device)
    calls = {
        "token_topk": lambda: ops.token_topk_decode(st["q"], st["kv"], st["indices"], st["indptr"], st["last"], ntok,
                                                     st["max_pages_used"], sink_tokens=sink, local_tokens=window,
                                                     out=st["out"], workspace=ws_tok),
        # strided overlapping blocks with the same budget: topk blocks of 16 tokens, a block every 8 tokens
        "strided_topk": lambda: ops.strided_topk_decode(st["q"], st["kv"], st["indices"], st["indptr"], st["last"], topk,
                                                         st["max_pages_used"], sink_tokens=sink, local_tokens=window,
                                                         out=st["out"], workspace=ws_str),
    }
    for name, call in calls.items():
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(nt)]
        with collector_paused():
            for _ in range(2):
                call()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for e0, e1 in evs:
                ops.append_paged_kv(st["k"], st["v"], st["kv"], None, st["indices"], st["indptr"], st["last"])
                e0.record()
                call()
                e1.record()
            torch.cuda.synchronize()
            tt = (time.perf_counter() - t0) / nt
        tks = [e0.elapsed_time(e1) for e0, e1 in evs]
        tk = statistics.fmean(tks) * 1e-3
        res[name] = {"sink_tokens": sink, "local_tokens": window, "ms_per_step": tt * 1e3, "value": B / tt,
                     "unit": "tokens/s", "steps": nt, "algorithmic_bytes_per_step": tok_bytes, "kernel_ms": tk * 1e3,
                     "kernel_ms_min": min(tks), "kernel_ms_max": max(tks), "achieved_gbs": tok_bytes / tk / 1e9,
                     "frac": tok_bytes / tk / 1e9 / HBM_PEAK_GBS, "traffic": traffic_of(name + "_kernel")}
    res["token_topk"]["topk_tokens"] = ntok
    res["strided_topk"].update(topk_blocks=topk, block_size=PS, stride=8)
    return res


def side_workload(torch, ops, name, steps, warmup, device, with_dense=True):
    """One of the other BASELINE configurations, measured like the headline:
    cache built, K steps timed, dense baseline on the same tensors, cache freed."""
    B, ctx, Hkv, G, topk, desc = WORKLOADS[name]
    st = build_state(torch, ops, B, ctx, Hkv, G, topk, device, ragged=name in RAGGED)
    torch.cuda.synchronize()
    ms_step, elapsed, kernel_ms, fused = time_step(torch, ops, st, B, Hkv, topk, steps, warmup)
    print(f"[bench] {name}: kv at {hex(st['kv'].data_ptr())}, kbar at {hex(st['kbar'].data_ptr())}, "
          f"{torch.cuda.memory_allocated() / 1e9:.1f} GB allocated, {torch.cuda.memory_reserved() / 1e9:.1f} GB reserved, "
          f"step {ms_step:.4f} ms, launches {min(LAST_LAUNCH_MS):.3f}..{max(LAST_LAUNCH_MS):.3f} ms "
          f"(first five {LAST_LAUNCH_MS[:5]}, last five {LAST_LAUNCH_MS[-5:]})", file=sys.stderr, flush=True)
    ab = algorithmic_bytes(st["lengths"], Hkv, G, topk)
    out = {"description": desc, "batch": B, "ctx": ctx, "num_kv_heads": Hkv, "num_q_heads": Hkv * G, "topk_pages": topk,
           "page_table": "ragged, half fragmented" if name in RAGGED else "reference layout p*B+b",
           "kv_resident_gb": round(st["kv"].numel() * 2 / 1e9, 2), "launches_per_step": len(kernel_ms),
           "steps": steps, "warmup": warmup, "ms_per_step": ms_step, "value": B * steps / elapsed, "unit": "tokens/s",
           "kernels_ms": kernel_ms, "algorithmic_bytes_per_step": ab["step"],
           "achieved_gbs": ab["step"] / (ms_step * 1e-3) / 1e9, "frac": ab["step"] / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBS}
    if LAST_GRAPH_REPLAY_MS is not None:
        # a step this short is host-bound when launched eagerly: the same launches replayed as one HIP graph
        out["graph_replay_ms_per_step"] = LAST_GRAPH_REPLAY_MS
        out["graph_replay_frac"] = ab["step"] / (LAST_GRAPH_REPLAY_MS * 1e-3) / 1e9 / HBM_PEAK_GBS
        out["graph_of_10_steps_replay_ms_per_step"] = LAST_GRAPH_REPLAY_10_MS
    if fused:
        out["kernel_frac"] = ab["step"] / (kernel_ms["fused_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS
        tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
        if os.path.exists(tpath):   # rocprofv3 counters of an earlier run of the same kernel and workload, not of this run
            with open(tpath) as f:
                out["traffic"] = json.load(f).get(f"{name}:B={B}", {}).get("blocktopk_step_kernel")
    if with_dense:
        td = time_dense(torch, ops, st, max(3, min(10, steps // 10)))
        out["dense_ms_per_step"] = td
        out["dense_frac"] = ab["dense"] / (td * 1e-3) / 1e9 / HBM_PEAK_GBS
        out["sparse_over_dense"] = td / ms_step
    # No empty_cache() here: the allocator keeps the freed blocks, and the next workload's cache is
    # carved from memory whose physical backing this process got first (returning it to the driver
    # and allocating again lands on a slower backing, 3-9 % on these kernels).
    del st
    return out


def manager_bench(torch, ops, steps, warmup, device):
    """The LiteSys-style KV manager (kinetics_amd/batch_cache.py, the paged stand-in for
    LiteSys/litesys/attention/batch_cache.py:86-168) around the fused step: wall time of one
    compute_attention call per layer -- offsets, page reservation and page table once per step,
    the kernels planned for the active sequences -- against the bare fused step on the same
    tensors.  Every slot is active; the block policy on every layer (attn_layer_skip=[])."""
    from types import SimpleNamespace

    from kinetics_amd.batch_cache import PagedBatchKVManager

    out = {}
    Hq, Hkv, topk, local = 4, 1, 64, 16
    # (layers: what fits beside the caches; the page table is built once per step, whatever their number)
    for B, ctx, L in ((32, 32768, 8), (256, 16384, 8), (4096, 8192, 4)):
        cfg = SimpleNamespace(num_attention_heads=Hq, num_key_value_heads=Hkv, head_dim=D, hidden_size=Hq * D, num_hidden_layers=L)
        m = PagedBatchKVManager(cfg, B, ctx + 1024, device, torch.bfloat16, attn_block_topk=topk, attn_local=local, attn_layer_skip=[])
        # state as after a prefill of ctx tokens per slot, written directly: offsets, pages, random K/V, mean keys
        gen = torch.Generator(device=device).manual_seed(7)
        lens = torch.full((B,), ctx + m.pad, dtype=torch.int32, device=device)
        m.pool.reserve(lens)
        idx = torch.empty(m.num_pool_pages, dtype=torch.int32, device=device)
        ptr = torch.empty(B + 1, dtype=torch.int32, device=device)
        last = torch.empty(B, dtype=torch.int32, device=device)
        m.pool.build_page_table(lens, idx, ptr, last)
        for layer in range(L):
            m.kv_offset[layer].fill_(ctx)
            kv = m.kv_cache[layer]
            chunk = max(1, (1 << 27) // (2 * m.page * Hkv * D))
            for s0 in range(0, kv.shape[0], chunk):
                e0 = min(kv.shape[0], s0 + chunk)
                kv[s0:e0] = torch.randn(e0 - s0, 2, m.page, Hkv, D, generator=gen, device=device).bfloat16()
            ops.build_kbar(kv, m.kbar[layer], idx, ptr, last)
        batch_idx = torch.arange(B, device=device)
        qs, ks, vs = (torch.randn(B, h, 1, D, generator=gen, device=device).bfloat16() for h in (Hq, Hkv, Hkv))

        def step():
            for layer in range(L):
                m.compute_attention(qs, ks, vs, layer, batch_idx)

        with collector_paused():
            for _ in range(warmup):
                step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                step()
            torch.cuda.synchronize()
            per_call = (time.perf_counter() - t0) / (steps * L)
        # the bare fused step on the manager's own tensors (table of the last step), layer after layer
        # like the manager (one layer's cache over and over would sit in the 256 MB last-level cache)
        n, slots, indptr, lastp = B, m._slots32[:B], m._indptr[: B + 1], m._last[:B]
        q3, k3, v3 = qs[:, :, 0, :], ks[:, :, 0, :], vs[:, :, 0, :]
        o3 = torch.empty_like(q3)

        def bare(layer):
            ops.blocktopk_decode_step(q3, k3, v3, m.kv_cache[layer], m.kbar[layer], m.page_indices, indptr, lastp, topk, out=o3,
                                      sink_pages=m.sink_pages, local_tokens=m.local_tokens, first_page_offset=m.pad,
                                      workspace=m._ws, slot_ids=slots)

        with collector_paused():
            for i in range(warmup):
                bare(i % L)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(steps * L):
                bare(i % L)
            torch.cuda.synchronize()
            per_bare = (time.perf_counter() - t0) / (steps * L)
        graph_ms = time_graph_replay(torch, step, steps, warmup) / L if per_call * 1e3 < GRAPH_REPLAY_BELOW_MS * 2 else None
        free, bits = m.pool.status()
        out[f"B={B}"] = {"batch": B, "ctx": ctx, "layers": L, "topk_pages": topk, "local_tokens": local,
                         "ms_per_layer_call": per_call * 1e3, "ms_bare_fused_step": per_bare * 1e3,
                         "glue_fraction": 1.0 - per_bare / per_call, "ms_per_layer_call_hip_graph": graph_ms,
                         "tokens_per_s_per_layer": B / per_call, "pool_status_bits": bits}
        print(f"[bench] manager B={B} ctx={ctx}: {per_call * 1e6:.1f} us per layer call, bare step {per_bare * 1e6:.1f} us, "
              f"glue {100 * (1 - per_bare / per_call):.1f} %" + (f", replayed as a graph {graph_ms * 1e3:.1f} us" if graph_ms else ""),
              file=sys.stderr, flush=True)
        del m, idx, ptr, last, qs, ks, vs
        torch.cuda.empty_cache()
    return out


def placement_rounds(torch, ops, args, B, ctx, Hkv, G, topk, device):
    """Same binary, same seeded inputs, several allocations of the cache in one
    process: round 0 is the process's first large allocation; later rounds reuse
    memory that was freed, behind a dummy allocation of varying size."""
    dummy_gib = [0, 0, 3, 11, 0, 27, 0, 5]
    rounds = []
    for r in range(args.placement_rounds):
        d = dummy_gib[r % len(dummy_gib)]
        dummy = torch.empty(d << 30, dtype=torch.uint8, device=device) if d else None
        st = build_state(torch, ops, B, ctx, Hkv, G, topk, device, ragged=args.workload in RAGGED)
        ms_step, _, kernel_ms, _ = time_step(torch, ops, st, B, Hkv, topk, max(5, min(args.steps, 20)), 3, args.mode)
        dense_ms = None if args.no_dense else time_dense(torch, ops, st, 3)
        rounds.append({"round": r, "dummy_gib": d, "kv_ptr": hex(st["kv"].data_ptr()), "ms_per_step": ms_step,
                       "kernels_ms": kernel_ms, "dense_ms_per_step": dense_ms})
        print(f"[placement] round {r}: dummy {d} GiB, kv at {hex(st['kv'].data_ptr())}, step {ms_step:.4f} ms, "
              f"dense {dense_ms if dense_ms is None else round(dense_ms, 3)} ms", file=sys.stderr, flush=True)
        del st, dummy
        torch.cuda.empty_cache()
    steps = [x["ms_per_step"] for x in rounds]
    return {"workload": args.workload, "batch": B, "placement_rounds": rounds,
            "ms_per_step_min": min(steps), "ms_per_step_max": max(steps), "spread": max(steps) / min(steps) - 1.0}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="qwen3-8b-share", choices=sorted(WORKLOADS) + ["custom"])
    ap.add_argument("--batch", type=int, default=0, help="override the workload's batch size")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-dense", action="store_true")
    ap.add_argument("--cpu-batch", type=int, default=128)
    ap.add_argument("--mode", default="auto", choices=["auto", "fused", "three"],
                    help="decode-step path: one fused launch, three launches (append / score+select / attention), "
                         "or what kinetics_amd.ops.prefer_fused_step picks for the shape")
    ap.add_argument("--whole-layer", action="store_true",
                    help="also time the whole decoder layer (norms, GEMMs, MLP around the attention path), "
                         "the quantity benchmark/blocktopk.py prints")
    ap.add_argument("--token-topk", action="store_true",
                    help="also time token-level top-k and strided-block decode (LiteSys' attn_topk / attn_stride "
                         "policies) with the same token budget; on by default for the headline workload")
    ap.add_argument("--no-side-workloads", action="store_true",
                    help="headline workload only: skip the `workloads` block (the other configurations) and the "
                         "token-granular policies")
    # the reference's own command line (benchmark/blocktopk.py:6-19, benchmark/README.md): a context of
    # gen_len / 2 tokens, the model's heads divided by world_size
    ap.add_argument("--model", default=None, help="e.g. Qwen/Qwen3-8B: build the workload from the reference's arguments")
    ap.add_argument("--gen_len", type=int, default=32768)
    ap.add_argument("--batch_size", type=int, default=256)
    ap.add_argument("--topk_page", type=int, default=64)
    ap.add_argument("--page_size", type=int, default=16, choices=[16, 32, 64, 128],
                    help="tokens per page of the cache (any workload; the reference's flag, benchmark/blocktopk.py:13)")
    ap.add_argument("--world_size", type=int, default=8)
    ap.add_argument("--head_dim", type=int, default=128, choices=[128, 64],
                    help="elements per head row (the reference reads it from the model config, "
                         "benchmark/blocktopk_decoder.py:104; every BASELINE configuration has 128)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float16"],
                    help="element type of q, the cache, the mean keys and the output (the reference's flag, "
                         "benchmark/blocktopk.py:18)")
    ap.add_argument("--placement-rounds", type=int, default=0,
                    help="instead of the benchmark: build, time (step and dense) and free the workload's cache this many "
                         "times in one process, with dummy allocations of varying size in front of it, to see how much "
                         "the physical placement of the cache moves the kernels; prints one JSON line")
    ap.add_argument("--manager", action="store_true",
                    help="instead of the benchmark: time the LiteSys-style KV manager's decode call per layer at 32 / 256 / 4096 "
                         "active slots against the bare fused step on the same tensors; prints one JSON line")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (known bytes) to scale profiler byte counters")
    args = ap.parse_args()
    global D
    D = args.head_dim
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the path is independent per (sequence, KV head) and is run on "
              "one GPU's share of the heads; --gpus above 1 is not supported.", file=sys.stderr)
        sys.exit(2)

    if args.model:
        from kinetics_amd.decoder_layer import qwen3_config

        mcfg = qwen3_config(args.model)
        hq, hkv = mcfg.num_attention_heads // args.world_size, mcfg.num_key_value_heads // args.world_size
        if hq < 1 or hkv < 1:
            print("bench.py: world_size exceeds the number of heads", file=sys.stderr)
            sys.exit(2)
        args.workload = "custom"
        WORKLOADS["custom"] = (args.batch_size, args.gen_len // 2 // args.page_size * args.page_size, hkv, hq // hkv, args.topk_page,
                               f"{args.model} at world_size {args.world_size}: {hkv} KV heads, {hq} Q heads")
        WHOLE_LAYER_MODEL["custom"] = (args.model, args.world_size)

    import torch

    from kinetics_amd import _lib, ops

    _lib.load()  # fail loudly if the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    device = torch.device("cuda:0")
    B, ctx, Hkv, G, topk, desc = WORKLOADS[args.workload]
    if args.batch:
        B = args.batch
    headline = args.workload == "qwen3-8b-share" and not args.batch
    if args.placement_rounds:
        print(json.dumps(placement_rounds(torch, ops, args, B, ctx, Hkv, G, topk, device)))
        return
    if args.manager:
        print(json.dumps({"manager": manager_bench(torch, ops, max(args.steps, 50), max(args.warmup, 10), device)}))
        return
    t_setup = time.perf_counter()
    page = args.page_size
    elem = torch.float16 if args.dtype == "float16" else torch.bfloat16
    st = build_state(torch, ops, B, ctx, Hkv, G, topk, device, ragged=args.workload in RAGGED, PS=page, dtype=elem)
    torch.cuda.synchronize()
    print(f"[bench] {args.workload}: B={B} ctx={ctx} H_kv={Hkv} G={G} topk={topk}, "
          f"KV {st['kv'].numel() * 2 / 1e9:.1f} GB resident at {hex(st['kv'].data_ptr())}, kbar at {hex(st['kbar'].data_ptr())}, "
          f"setup {time.perf_counter() - t_setup:.1f}s", file=sys.stderr, flush=True)

    # -- the timed region: K steps between two synchronisations and two HIP events on the launch stream
    K = args.steps
    ms_step, elapsed, kernel_ms, fused = time_step(torch, ops, st, B, Hkv, topk, K, args.warmup, args.mode)

    ab = algorithmic_bytes(st["lengths"], Hkv, G, topk, page)
    step_gbs = ab["step"] / (ms_step * 1e-3) / 1e9
    if fused:
        dom_name, dom_kernel, dom_bytes, dom_ms = ("blocktopk_step_kernel (append + score + select + attention, fused)",
                                                   "blocktopk_step_kernel", ab["step"], kernel_ms["fused_step"])
    else:
        dom_name, dom_kernel, dom_bytes, dom_ms = ("paged_decode_kernel (sparse gather-attention)",
                                                   "paged_decode_kernel", ab["attention"], kernel_ms["sparse_attention"])
        kernel_ms["score_topk_gbs"] = ab["score_select"] / (kernel_ms["score_topk"] * 1e-3) / 1e9
    dom_gbs = dom_bytes / (dom_ms * 1e-3) / 1e9
    traffic_table = {}
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            traffic_table = json.load(f).get(f"{args.workload}:B={B}", {})
    traffic = traffic_table.get(dom_kernel)
    world, layers = REFERENCE_NORMALISATION.get(args.workload, (None, None))

    result = {
        "metric": "decode tok/s per layer, Qwen3-8B 1-GPU share B=4096 ctx=32K; HBM GB/s % peak",
        "value": B * K / elapsed,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if elem is torch.bfloat16 else "f16",
        "data": "synthetic",
        "config": {"workload": args.workload, "description": desc, "batch": B, "ctx": ctx, "num_kv_heads": Hkv,
                   "num_q_heads": Hkv * G, "head_dim": D, "page_size": page, "topk_pages": topk,
                   "page_table": "ragged, half fragmented" if args.workload in RAGGED else "reference layout p*B+b",
                   "kv_resident_gb": round(st["kv"].numel() * 2 / 1e9, 2),
                   "launches_per_step": len(kernel_ms) - (0 if fused else 1)},
        "roofline": {"bound": "hbm", "kernel": dom_name,
                     "achieved": dom_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dom_gbs / HBM_PEAK_GBS,
                     "traffic": traffic,
                     "traffic_source": ("profiles/hbm_traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run "
                                        "of this kernel on this workload, scaled by a 1 GiB copy; not measured by this run")
                     if traffic is not None else None,
                     "algorithmic_bytes_per_launch": dom_bytes,
                     "avg_launch_ms": dom_ms},
        "step_hbm": {"algorithmic_bytes_per_step": ab["step"], "bytes_per_seq": ab["per_seq"], "achieved": step_gbs,
                     "unit": "GB/s", "frac": step_gbs / HBM_PEAK_GBS},
        "kernels_ms": kernel_ms,
    }
    if LAST_GRAPH_REPLAY_MS is not None:
        result["graph_replay_ms_per_step"] = LAST_GRAPH_REPLAY_MS
        result["graph_replay_frac"] = ab["step"] / (LAST_GRAPH_REPLAY_MS * 1e-3) / 1e9 / HBM_PEAK_GBS
        result["graph_of_10_steps_replay_ms_per_step"] = LAST_GRAPH_REPLAY_10_MS
    if world:
        # the figure benchmark/blocktopk.py:82 prints divides the per-layer rate by world_size * num_hidden_layers;
        # it is built from the attention step alone here (the whole layer: --whole-layer)
        result["normalised_like_reference_print"] = {
            "value": B * K / elapsed / (world * layers), "unit": "tokens/s", "world_size": world, "num_hidden_layers": layers,
            "note": "attention step only / (world_size * num_hidden_layers), cf. benchmark/blocktopk.py:82"}

    if args.calibrate_copy:
        src = torch.empty(1 << 29, dtype=torch.bfloat16, device=device).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if not args.no_dense:
        nd = max(3, min(10, K // 10))
        td = time_dense(torch, ops, st, nd) * 1e-3
        dense_bytes = ab["dense"]
        result["dense_baseline"] = {"value": B / td, "unit": "tokens/s", "ms_per_step": td * 1e3, "steps": nd,
                                    "achieved_gbs": dense_bytes / td / 1e9, "frac": dense_bytes / td / 1e9 / HBM_PEAK_GBS,
                                    "sparse_over_dense": (B * K / elapsed) / (B / td)}
    side = headline and page == PS and elem is torch.bfloat16 and not args.no_side_workloads
    if (args.token_topk or side) and page == PS and elem is torch.bfloat16:   # token-granular policies: 16-token pages, bf16
        result.update(time_token_policies(torch, ops, st, B, Hkv, G, topk, max(3, min(20, K // 5)), traffic_table.get))
    del st
    if not side:
        torch.cuda.empty_cache()
    if side:
        # every other BASELINE configuration in the same run, each on its own freshly built cache
        # (carved from the blocks the headline cache has just left in the allocator)
        # whatever --steps / --warmup the headline was given: at least 100 timed steps after at least 20
        # warm-ups each (they cost under 0.1 s per workload; the reference warms up 200 times,
        # benchmark/blocktopk.py:49)
        ks, ws = max(100, K), max(20, args.warmup)
        result["workloads"] = {name: side_workload(torch, ops, name, ks, ws, device)
                               for name in ("qwen3-8b-tp1", "qwen3-0.6b-mix", "qwen3-32b-share", "qwen3-8b-readme", "tiny")}
        torch.cuda.empty_cache()
    if args.whole_layer and args.workload in WHOLE_LAYER_MODEL:
        result["whole_layer"] = whole_layer(torch, args, B, ctx, topk, device)
    if not args.no_cpu_baseline and Hkv == 1 and args.workload not in RAGGED:
        result["cpu_baseline"] = cpu_baseline(torch, min(args.cpu_batch, B), ctx, G, topk)
        if side:
            tb, tctx, _, tg, tk, _ = WORKLOADS["tiny"]
            result["cpu_baseline"]["tiny_in_full"] = cpu_baseline(torch, tb, tctx, tg, tk, budget_s=3.0)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
