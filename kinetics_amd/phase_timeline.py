"""Per-phase timeline of the fused decode step, from clock stamps inside the kernel.

    python3 -m kinetics_amd.phase_timeline --workload qwen3-8b-readme
    python3 -m kinetics_amd.phase_timeline --workload qwen3-8b-share --batch 8 --topk 2048

Loads the diagnostic twin of the library (``libkinetics_amd_phases.so``: the same sources
compiled with ``-DKIN_TUNE``, in which thread 0 of each of the first 1024 workgroups of
``blocktopk_step_kernel`` records a 100 MHz clock value at every phase boundary), runs one
of bench.py's workloads and prints, for every boundary, when the workgroups pass it
(minimum / median / maximum over the workgroups, in microseconds since the first one
started) and how long they spend between consecutive boundaries.  The stamps cost a few
hundred nanoseconds per workgroup; the operators never load this build.
"""
from __future__ import annotations

import argparse
import ctypes
import os
import statistics
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# tag -> what has happened when the stamp is taken (kin_step.hip, kin_select.h)
PHASES = {
    0: "workgroup starts",
    1: "table entries of the sequence read",
    2: "new token appended",
    40: "team: slice of the mean keys requested",
    41: "team: slice scored, keys stored for the team",
    42: "team: every member's keys stored (or patience over)",
    43: "team: the list's keys loaded into LDS",
    17: "mean keys start to stream",
    16: "mean query in registers",
    18: "last mean key scored",
    19: "scores in LDS",
    20: "select starts",
    21: "radix digit 0 fixed",
    22: "radix digit 1 fixed",
    23: "radix digit 2 fixed",
    24: "radix digit 3 fixed",
    25: "winners gathered",
    30: "page list ready",
    31: "pages attended",
    44: "team: partial result stored, counted in",
    45: "team: parts merged, output written",
    # the token-granular policies (kin_token_topk.hip)
    50: "token policy: this workgroup's tokens scored",
    51: "token policy: every share scored, select starts",
    54: "token policy: keys requested",
    55: "token policy: radix digit 0 fixed",
    56: "token policy: radix digit 1 fixed",
    57: "token policy: radix digit 2 fixed",
    58: "token policy: radix digit 3 fixed",
    59: "token policy: winners listed in position order",
    52: "token policy: token list ready",
    53: "token policy: listed tokens attended",
}
MAX_WGS, MAX_STAMPS = 1024, 64


def main() -> None:
    import numpy as np
    import torch

    import bench
    from kinetics_amd import _lib, ops
    from kinetics_amd.build import PHASES_LIB_PATH, build_phases_library

    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--workload", default="qwen3-8b-readme", choices=sorted(bench.WORKLOADS))
    ap.add_argument("--batch", type=int, default=None, help="override the workload's batch size")
    ap.add_argument("--topk", type=int, default=None, help="override the workload's page budget")
    ap.add_argument("--policy", default="block", choices=["block", "token", "strided"],
                    help="block: the fused block top-k step; token / strided: LiteSys' token-granular policies "
                         "(token budget 16 x the page budget, 4 sink tokens, a local window of 16)")
    ap.add_argument("--warmup", type=int, default=10)
    args = ap.parse_args()
    if not PHASES_LIB_PATH.exists():
        build_phases_library(verbose=False)
    lib = ctypes.CDLL(str(PHASES_LIB_PATH))
    for name, (restype, argtypes) in _lib.SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = restype, argtypes
    accessor = lib.kin_debug_stamps_step if args.policy == "block" else lib.kin_debug_stamps_token
    accessor.restype = ctypes.c_int
    accessor.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    _lib._lib = lib  # this process only: the operators below call the diagnostic build

    B, ctx, Hkv, G, topk, _ = bench.WORKLOADS[args.workload]
    B = args.batch or B
    topk = args.topk or topk
    dev = "cuda"
    st = bench.build_state(torch, ops, B, ctx, Hkv, G, topk, dev, ragged=args.workload in bench.RAGGED)
    ws = torch.empty(max(16, ops.step_workspace_bytes(B, Hkv, st["kbar"].shape[2])), dtype=torch.uint8, device=dev)

    max_pages = st["max_pages_used"]
    if args.policy == "token":
        ws = torch.empty(max(16, ops.token_topk_workspace_bytes(B, Hkv, max_pages)), dtype=torch.uint8, device=dev)
    elif args.policy == "strided":
        ws = torch.empty(max(16, ops.strided_topk_workspace_bytes(B, Hkv, max_pages)), dtype=torch.uint8, device=dev)

    def step():
        if args.policy == "token":
            ops.token_topk_decode(st["q"], st["kv"], st["indices"], st["indptr"], st["last"], 16 * topk, max_pages, sink_tokens=4,
                                  local_tokens=16, out=st["out"], workspace=ws)
        elif args.policy == "strided":
            ops.strided_topk_decode(st["q"], st["kv"], st["indices"], st["indptr"], st["last"], topk, max_pages, block_size=16,
                                    stride=8, sink_tokens=4, local_tokens=16, out=st["out"], workspace=ws)
        else:
            ops.blocktopk_decode_step(st["q"], st["k"], st["v"], st["kv"], st["kbar"], st["indices"], st["indptr"], st["last"], topk,
                                      out=st["out"], workspace=ws)

    stamps = np.zeros(MAX_WGS * MAX_STAMPS * 2, dtype=np.int64)
    counts = np.zeros(MAX_WGS, dtype=np.int32)

    def read():
        rc = accessor(stamps.ctypes.data_as(ctypes.c_void_p), counts.ctypes.data_as(ctypes.c_void_p))
        if rc != 0:
            raise RuntimeError(f"reading the stamps failed ({rc})")

    for _ in range(args.warmup):
        step()
    read()  # empties the stamps of the warm-up
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    reps = 10
    e0.record()
    for _ in range(reps):
        step()
    e1.record()
    read()  # the stamps of the last of these launches (every workgroup starts by emptying its own)
    table = stamps.reshape(MAX_WGS, MAX_STAMPS, 2)
    wgs = [w for w in range(MAX_WGS) if counts[w] > 0]
    t0 = min(int(table[w, 0, 1]) for w in wgs)
    lists = B * Hkv
    print(f"== {args.workload}{'' if args.policy == 'block' else ' (' + args.policy + ' policy)'}: batch {B}, {Hkv} KV x {G} Q heads, ctx {ctx}, {topk} pages per list: {lists} lists; "
          f"{len(wgs)} workgroups stamped{' (the first 1024)' if len(wgs) == MAX_WGS else ''}; "
          f"{e0.elapsed_time(e1) * 1e3 / reps:.1f} us per launch by HIP events, {reps} launches back to back")
    print("   when the workgroups pass each boundary (us since the first workgroup started):")
    for tag, what in PHASES.items():
        ts = [(int(table[w, i, 1]) - t0) / 100.0 for w in wgs for i in range(counts[w]) if table[w, i, 0] == tag]
        if ts:
            print(f"   {what:52s} n={len(ts):5d}  min {min(ts):7.1f}  median {statistics.median(ts):7.1f}  max {max(ts):7.1f}")
    print("   time between consecutive boundaries of a workgroup (us):")
    durs: dict = {}
    for w in wgs:
        for i in range(1, counts[w]):
            key = (int(table[w, i - 1, 0]), int(table[w, i, 0]))
            durs.setdefault(key, []).append((int(table[w, i, 1]) - int(table[w, i - 1, 1])) / 100.0)
    order = list(PHASES)
    for key in sorted(durs, key=lambda k: (order.index(k[1]) if k[1] in order else 99, order.index(k[0]) if k[0] in order else 99)):
        d = durs[key]
        a, b = PHASES.get(key[0], str(key[0])), PHASES.get(key[1], str(key[1]))
        print(f"   {a:52s} -> {b:52s} n={len(d):5d}  mean {statistics.mean(d):6.2f}  median {statistics.median(d):6.2f}  max {max(d):6.2f}")


if __name__ == "__main__":
    main()
