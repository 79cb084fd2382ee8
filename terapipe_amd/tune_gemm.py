"""Measures every tile configuration x k-split of ``tp_gemm`` on the GEMM shapes of a layer geometry and writes
the winners to ``csrc/gemm_tuned.inc``, the table ``plan_gemm`` consults before its heuristics.

    python -m terapipe_amd.tune_gemm --geometry 2048:8192:256:2048 --geometry 5120:20480:512,384,...:2048 ...

A geometry is ``hidden:ffn:slice_tokens[,slice_tokens...]:step_tokens``: the forward GEMMs (NT) and data-gradient
GEMMs (NN) are measured at every ``slice_tokens`` (tokens of a slice x batch), the parameter-gradient GEMMs
(TN) at ``step_tokens`` (all tokens of a step).  Weights rotate through a set larger than the caches so that
they stream from HBM as they do in a step.  Needs the GPU, and a library built with an empty table (the
heuristic plan is the yardstick); rebuild the library afterwards.

    python -m terapipe_amd.tune_gemm --in-step 2048:8192:16:24:1:256,256,256,256,256,256,256,256

searches in the step itself instead (``hidden:ffn:heads:layers:batch:slice_tokens,...``): the runner runs whole
forward + backward steps with three slice streams and launch replay, and one slice GEMM shape at a time is given
every plan in turn (``ops.GEMM_PLAN_OVERRIDE``); a plan is kept when it shortens the step.  It starts from the
table that is compiled in and prints the entries to change.  This is the measure that counts when launches
overlap: the fastest plan for a GEMM alone on the chip is often not the one that shares it best.
"""
import argparse
import os
import sys

import torch

from . import _lib, ops

DEFAULT_GEOMETRIES = [
    "2048:8192:256:2048",                                   # GPT-3 1.3B shape, 256-token slices
    "5120:20480:512,384,320,256,224,192,160:2048",          # 13B shape, DP-style slices
    "12288:49152:128:2048",                                 # 175B shape, 128-token slices
    "6144:24576:64:4096",                                   # 44B shape, 32-token slices x batch 2
]
DMA_CFGS = [2, 3, 5, 6, 7, 8, 10, 11, 12, 13, 14, 15, 16, 17, 18, 19, 20, 41, 42, 43]
# the weight-streaming kernel's configurations (NT and NN only; 24 and 25 NT only): cfg -> rows of its row tile
STREAM_CFGS = {21: 192, 22: 256, 24: 192, 25: 256, 26: 128, 29: 256, 30: 192, 31: 192, 32: 256, 33: 192, 34: 256,
               35: 128, 36: 64, 37: 128, 38: 64}
SPLITS = [1, 2, 3, 4, 6, 8]
# k splits the in-step search tries (the library deals whole k-tiles to the splits, evenly to within one).  Inside a step the slice streams share the
# chip, and fewer splits than are fastest for a launch alone often win: fewer, larger workgroups and fewer partial sums.
IN_STEP_SPLITS = (1, 2, 3, 4, 5, 6, 8)
OPS = {"NT": _lib.TP_GEMM_NT, "NN": _lib.TP_GEMM_NN, "TN": _lib.TP_GEMM_TN}


_PAIR_STREAMS = []


def _time_pair_us(fn, n=6):
    """Two chains of the same call on two streams inside one graph: time per call when a neighbour shares the GPU
    (the runner overlaps consecutive slices on two streams)."""
    while len(_PAIR_STREAMS) < 2:
        _PAIR_STREAMS.append(torch.cuda.Stream())
    s0, s1 = _PAIR_STREAMS
    fn(0, 0)
    fn(1, 1)
    torch.cuda.synchronize()
    with torch.cuda.stream(s0):
        fn(0, 0)
    with torch.cuda.stream(s1):
        fn(1, 1)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        main = torch.cuda.current_stream()
        s1.wait_stream(main)
        with torch.cuda.stream(s1):
            for i in range(n):
                fn(2 * i + 1, 1)
        for i in range(n):
            fn(2 * i, 0)
        main.wait_stream(s1)
    g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    g.replay()
    g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / (4 * n) * 1e3


_WARMUP_STREAM = []


def _time_us(fn, n=6):
    fn(0)
    torch.cuda.synchronize()
    # one side stream for every call: the library's workspaces are per stream and never shrink
    if not _WARMUP_STREAM:
        _WARMUP_STREAM.append(torch.cuda.Stream())
    side = _WARMUP_STREAM[0]
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn(1)
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(n):
            fn(i)
    g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    g.replay()
    g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / (2 * n) * 1e3


def sweep(op, M, N, K, dtype, device, log, pair=False):
    """Returns (best_us, cfg, nsplit, automatic_us) for one shape."""
    a_shape = (K, M) if op == "TN" else (M, K)
    b_shape = (N, K) if op == "NT" else (K, N)
    nb = max(2, min(8, int(1.0e9 // (N * K * 2))))
    A = torch.randn(a_shape, device=device, dtype=dtype)
    Bs = [torch.randn(b_shape, device=device, dtype=dtype) for _ in range(nb)]
    C = torch.empty(M, N, device=device, dtype=dtype)
    code = OPS[op]
    if pair:
        Cs = [C, torch.empty_like(C)]
        time_it = lambda **kw: _time_pair_us(lambda i, lane: ops.gemm(code, A, Bs[i % nb], M, N, K, C=Cs[lane], **kw))
    else:
        time_it = lambda **kw: _time_us(lambda i: ops.gemm(code, A, Bs[i % nb], M, N, K, C=C, **kw))
    auto = time_it()
    results = []
    for cfg in DMA_CFGS + (sorted(STREAM_CFGS) if op != "TN" and K % 64 == 0 else []):
        for ns in SPLITS:
            if K // ns < 512 or (17 <= cfg <= 20 and (M < 192 or K % 64)) or (cfg == 17 and op != "NT"):
                continue
            if cfg in (2, 6, 7, 14, 15, 16) and (K % 64 or (cfg == 14 and op == "TN") or (cfg in (6, 7) and op != "NT") or
                                                 (cfg in (2, 6, 7, 14, 15) and M < 128)):
                continue
            if cfg in (41, 42, 43) and (K % 64 or op == "TN" or (cfg == 43 and op != "NT") or M < 128):
                continue
            if cfg in STREAM_CFGS and ((cfg in (24, 25) and op != "NT") or STREAM_CFGS[cfg] < M // 2 or
                                       STREAM_CFGS[cfg] >= 2 * M):
                continue
            try:
                t = time_it(tile_cfg=cfg, ksplit=ns)
            except _lib.TeraPipeHipError:
                continue
            results.append((t, cfg, ns))
    results.sort()
    best = results[0]
    print("%s %dx%dx%d: automatic %.1f us | %s" % (op, M, N, K, auto, "  ".join(
        "c%d/s%d:%.1f" % (c, s, t) for t, c, s in results[:5])), file=log, flush=True)
    return best[0], best[1], best[2], auto


def shapes_of(geometry):
    E, F, slices, step = geometry.split(":")
    E, F, step = int(E), int(F), int(step)
    out = []
    for N, K in ((3 * E, E), (E, E), (F, E), (E, F)):
        for M in sorted({int(v) for v in slices.split(",")}):
            out.append(("NT", M, N, K))
            out.append(("NN", M, K, N))        # dX = dY[M, N] @ W[N, K]
        out.append(("TN", N, K, step))         # dW[N, K] = dY[step, N]^T @ X[step, K]
    return out


def in_step(spec, dtype=torch.float16, log=sys.stderr, only_rows=None, only_cfgs=None):
    """Coordinate descent over the plans of the slice GEMMs (NT forward, NN data gradient) of one geometry,
    timing whole steps.  Returns [(op, M, N, K, cfg, nsplit)] for the shapes whose plan changed."""
    import time
    from . import TeraPipe, TransformerLayers
    E, F, H, n_layers, B, slices = spec.split(":")
    E, F, H, n_layers, B = int(E), int(F), int(H), int(n_layers), int(B)
    slices = [int(v) for v in slices.split(",")]
    L = sum(slices)
    device = torch.device("cuda:0")
    layers = TransformerLayers(n_layers, E, F, H, dtype=dtype, device=device)
    g = torch.Generator(device="cpu").manual_seed(0)
    with torch.no_grad():
        for p in layers.parameters():
            if p.dim() == 2:
                p.copy_((torch.randn(p.shape, generator=g) * 0.02).to(dtype))
    runner = TeraPipe(layers, B, L, [B], slices, slice_streams=3, launch_replay=True)
    x = torch.randn(L, B, E, generator=g).to(dtype).to(device)
    R = torch.randn(L, B, E, generator=g).to(dtype).to(device)

    def one_step():
        for p in layers.parameters():
            p.grad = None
        (runner(x) * R).sum().backward()

    def step_ms(n):
        if runner._sbufs is not None:       # record the launches again under the current overrides
            runner._sbufs.fwd_program = runner._sbufs.bwd_program = 0
        for _ in range(3):
            one_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            one_step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e3

    base = min(step_ms(8), step_ms(8))
    print("step with the compiled-in plans: %.2f ms" % base, file=log, flush=True)
    shapes = []
    for N, K in ((3 * E, E), (E, E), (F, E), (E, F)):
        for M in sorted({t * B for t in slices}):
            if only_rows is None or M in only_rows:
                shapes += [("NT", M, N, K), ("NN", M, K, N)]
    chosen = {}
    for op, M, N, K in shapes:
        key = (OPS[op], M, N, K)
        trials = []
        for cfg in (only_cfgs or DMA_CFGS):
            for ns in IN_STEP_SPLITS:
                if K // ns < 512 or (17 <= cfg <= 20 and (M < 192 or K % 64)) or (cfg == 17 and op != "NT"):
                    continue
                if cfg in (2, 6, 7, 14, 15, 16) and (K % 64 or (cfg in (6, 7) and op != "NT") or
                                                     (cfg in (2, 6, 7, 14, 15) and M < 128)):
                    continue
                if cfg in (41, 42, 43) and (K % 64 or (cfg == 43 and op != "NT") or M < 128):
                    continue
                ops.GEMM_PLAN_OVERRIDE[key] = (cfg, ns)
                try:
                    trials.append((step_ms(4), cfg, ns))
                except _lib.TeraPipeHipError:
                    pass
        trials.sort()
        ops.GEMM_PLAN_OVERRIDE.pop(key, None)
        pick, pick_ms = None, min(step_ms(8), step_ms(8))
        for _, cfg, ns in trials[:2]:           # confirm against the incumbent with longer runs
            ops.GEMM_PLAN_OVERRIDE[key] = (cfg, ns)
            t = min(step_ms(8), step_ms(8))
            if t < 0.995 * pick_ms:
                pick, pick_ms = (cfg, ns), t
        if pick is None:
            ops.GEMM_PLAN_OVERRIDE.pop(key, None)
        else:
            ops.GEMM_PLAN_OVERRIDE[key] = pick
            chosen[(op, M, N, K)] = pick + (pick_ms,)
        print("%s %dx%dx%d: %s -> step %.2f ms" % (op, M, N, K, pick or "unchanged", pick_ms), file=log, flush=True)
    print("step with the picks: %.2f ms" % min(step_ms(8), step_ms(8)), file=log, flush=True)
    return [(op, M, N, K, c, ns, ms) for (op, M, N, K), (c, ns, ms) in chosen.items()]


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--geometry", action="append")
    ap.add_argument("--out", default=os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "gemm_tuned.inc"))
    ap.add_argument("--in-step", metavar="SPEC",
                    help="hidden:ffn:heads:layers:batch:slice_tokens,... -- search the slice GEMM plans by timing "
                         "whole steps; prints the table entries to change")
    ap.add_argument("--only-rows", metavar="M,M,...",
                    help="with --in-step: search only the slice GEMMs of these row counts (a whole geometry can take "
                         "longer than one sitting)")
    ap.add_argument("--only-cfgs", metavar="C,C,...",
                    help="with --in-step: try only these tile configurations (the incumbent plan stays the yardstick)")
    ap.add_argument("--pair", action="store_true",
                    help="time two concurrent chains of each GEMM on two streams (per-call time with a neighbour) "
                         "instead of one chain alone")
    ap.add_argument("--min-gain", type=float, default=0.03,
                    help="shapes whose best time is within this fraction of the heuristic plan's get no entry")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        sys.exit("tune_gemm: needs the GPU")
    if args.in_step:
        rows = {int(v) for v in args.only_rows.split(",")} if args.only_rows else None
        cfgs = [int(v) for v in args.only_cfgs.split(",")] if args.only_cfgs else None
        for op, M, N, K, cfg, ns, ms in in_step(args.in_step, only_rows=rows, only_cfgs=cfgs):
            print("{TP_GEMM_%s, %d, %d, %d, %d, %d},  // in-step search: step %.2f ms" % (op, M, N, K, cfg, ns, ms))
        return
    device = torch.device("cuda:0")
    seen, rows = set(), []
    for geo in args.geometry or DEFAULT_GEOMETRIES:
        for shape in shapes_of(geo):
            if shape in seen:
                continue
            seen.add(shape)
            op, M, N, K = shape
            t, cfg, ns, auto = sweep(op, M, N, K, torch.float16, device, sys.stderr, pair=args.pair and op != "TN")
            rows.append((op, M, N, K, cfg, ns, t, auto))
    with open(args.out, "w") as f:
        f.write("// Measured best tile configuration and k-split per shape on MI355X (fp16; written by\n"
                "// terapipe_amd/tune_gemm.py).  {op, M, N, K, cfg, nsplit}  // best us, heuristic plan's us\n"
                "// (entries within %g %% of the heuristic plan are left to the heuristics)\n" % (100 * args.min_gain))
        for op, M, N, K, cfg, ns, t, auto in sorted(rows):
            if t >= (1.0 - args.min_gain) * auto:
                continue
            f.write("{TP_GEMM_%s, %d, %d, %d, %d, %d},  // %.1f  %.1f\n" % (op, M, N, K, cfg, ns, t, auto))
    print("wrote %d entries to %s" % (len(rows), args.out))


if __name__ == "__main__":
    main()
