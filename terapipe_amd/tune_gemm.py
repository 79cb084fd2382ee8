"""Measures every tile configuration x k-split of ``tp_gemm`` on the GEMM shapes of a layer geometry and writes
the winners to ``csrc/gemm_tuned.inc``, the table ``plan_gemm`` consults before its heuristics.

    python -m terapipe_amd.tune_gemm --geometry 2048:8192:256:2048 --geometry 5120:20480:512,384,...:2048 ...

A geometry is ``hidden:ffn:slice_tokens[,slice_tokens...]:step_tokens``: the forward GEMMs (NT) and data-gradient
GEMMs (NN) are measured at every ``slice_tokens`` (tokens of a slice x batch), the parameter-gradient GEMMs
(TN) at ``step_tokens`` (all tokens of a step).  Weights rotate through a set larger than the caches so that
they stream from HBM as they do in a step.  Needs the GPU, and a library built with an empty table (the
heuristic plan is the yardstick); rebuild the library afterwards.
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
DMA_CFGS = [3, 5, 8, 10, 11, 12, 13, 17, 18, 19, 20]
SPLITS = [1, 2, 3, 4, 6, 8]
OPS = {"NT": _lib.TP_GEMM_NT, "NN": _lib.TP_GEMM_NN, "TN": _lib.TP_GEMM_TN}


def _time_pair_us(fn, n=6):
    """Two chains of the same call on two streams inside one graph: time per call when a neighbour shares the GPU
    (the runner overlaps consecutive slices on two streams)."""
    s0, s1 = torch.cuda.Stream(), torch.cuda.Stream()
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


def _time_us(fn, n=6):
    fn(0)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
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
    for cfg in DMA_CFGS:
        for ns in SPLITS:
            if K // ns < 512 or (cfg >= 17 and (M < 192 or K % 64)) or (cfg == 17 and op != "NT"):
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


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--geometry", action="append")
    ap.add_argument("--out", default=os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "gemm_tuned.inc"))
    ap.add_argument("--pair", action="store_true",
                    help="time two concurrent chains of each GEMM on two streams (per-call time with a neighbour) "
                         "instead of one chain alone")
    ap.add_argument("--min-gain", type=float, default=0.03,
                    help="shapes whose best time is within this fraction of the heuristic plan's get no entry")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        sys.exit("tune_gemm: needs the GPU")
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
