#!/usr/bin/env python3
"""Headline benchmark: sliced GPT-layer-stack forward + reverse-slice backward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3|C2|C4|C5|C1]
    python bench.py --attention-grid            # the (T, P) micro-grid of the prefix-attention kernels

One step = every sequence slice of one synthetic batch through the whole layer stack forward (K/V
caches growing slice by slice), then the reverse-order slice backward, with the loss
``sum(y * R)`` for a fixed random R (inputs N(0,1), weights N(0,0.02), all resident in HBM before the
timed region).  Prints ONE JSON line: tokens/s of the workload (default C3, the GPT-3 13B stage share),
the MFMA roofline of its GEMM kernels (algorithmic flops / kernel time, measured live: the GEMM calls
of one recorded step replayed in a HIP graph between two HIP events; also per GEMM shape next to the
bound min(MFMA peak, operand bytes / HBM peak) allows), the HBM figure of the prefix-attention
kernels of the 32-token-slice workload C5, the same figures in short for the other 16-bit workloads, and
the CPU oracle timed on this host's cores on a bounded sample.
"""
import argparse
import gc
import json
import os
import re
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published peaks
PEAK_MFMA_16BIT = 2.5e15     # dense fp16/bf16 MFMA flop/s
PEAK_MFMA_FP32 = 157.3e12
PEAK_HBM = 8.0e12            # bytes/s

WORKLOADS = {
    # name: layers, hidden, heads, ffn, seq, batch, dtype, slices, weight std
    "C1": dict(desc="tiny GPT stack fp32: 4 layers, hidden 256, 4 heads, FFN 1024, seq 128, batch 2, 8x16 slices",
               n_layers=4, E=256, H=4, F=1024, L=128, B=2, dtype="f32", slices=[16] * 8, std=0.02),
    "C2": dict(desc="GPT-3 1.3B shape: 24 layers, hidden 2048, 16 heads, FFN 8192, seq 2048, batch 1, fp16, 8x256 slices",
               n_layers=24, E=2048, H=16, F=8192, L=2048, B=1, dtype="f16", slices=[256] * 8, std=0.02,
               streams=4),     # its slice GEMMs are 32-128 tiles each: four lanes measured 7 % faster than three
    "C3": dict(desc="GPT-3 13B stage share: 5 layers, hidden 5120, 40 heads, FFN 20480, seq 2048, batch 1, fp16, "
                    "slices [512,384,320,256,224,192,160]",
               n_layers=5, E=5120, H=40, F=20480, L=2048, B=1, dtype="f16",
               slices=[512, 384, 320, 256, 224, 192, 160], std=0.02),
    "C4": dict(desc="GPT-3 175B stage share: 2 layers, hidden 12288, 96 heads, FFN 49152, seq 2048, batch 1, bf16, 16x128 slices",
               n_layers=2, E=12288, H=96, F=49152, L=2048, B=1, dtype="bf16", slices=[128] * 16, std=0.006),
    "C5": dict(desc="GPT-3 44B stage share: 4 layers, hidden 6144, 48 heads, FFN 24576, seq 2048, batch 2, bf16, 64x32 slices",
               n_layers=4, E=6144, H=48, F=24576, L=2048, B=2, dtype="bf16", slices=[32] * 64, std=0.02),
}
TORCH_DTYPE = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
GEMM_OPS = {0: "NT", 1: "NN", 2: "TN"}


def gemm_flops_per_step(w):
    """72 * E^2 flops per token per layer fwd+bwd for F = 4E; stated generally as
    3 passes (fwd, dX, dW) x 2 * (3E*E + E*E + 2*E*F) per token."""
    per_token_fwd = 2 * (3 * w["E"] * w["E"] + w["E"] * w["E"] + 2 * w["E"] * w["F"])
    return 3 * per_token_fwd * w["L"] * w["B"] * w["n_layers"]


def attn_bytes_per_call(es, B, H, E, T, P, bwd):
    """Algorithmic HBM bytes of one prefix-attention call (one layer, one slice): elements x dtype size
    plus the fp32 LSE / delta vectors.  fwd (2T + 2S) B E; bwd (6T + 2S + 4P) B E."""
    S, BE, BH = P + T, B * E, B * H
    if not bwd:
        return (2 * T + 2 * S) * BE * es + 4 * BH * T
    return (6 * T + 2 * S + 4 * P) * BE * es + 8 * BH * T


def gemm_shape_work(meta, es):
    """(flops, algorithmic bytes) of one recorded GEMM call: a single (op, M, N, K) or, for a grouped launch,
    a tuple of them.  Bytes: both operands in once, the result out once."""
    metas = meta if isinstance(meta[0], tuple) else (meta,)
    flops = sum(2 * M * N * K for (_, M, N, K) in metas)
    nbytes = sum((M * K + N * K + M * N) * es for (_, M, N, K) in metas)
    return flops, nbytes


def gemm_shape_name(meta):
    metas = meta if isinstance(meta[0], tuple) else (meta,)
    return " + ".join("%s %dx%dx%d" % (GEMM_OPS[op], M, N, K) for (op, M, N, K) in metas)


def pmc_traffic(workload):
    """Bytes per GEMM launch of a step between L2 and the fabric, from the committed summary of the two rocprofv3 --pmc
    runs (FETCH_SIZE, WRITE_SIZE, each scaled by its reading on kernels of known size) over one step of this workload;
    None when no such summary is in the tree."""
    path = os.path.join(ROOT, "profiles", "bench_%s_gemm_hbm_traffic.pmc.txt" % workload)
    try:
        m = re.search(r"traffic_bytes_per_gemm_launch:\s*([0-9.eE+]+)", open(path).read())
    except OSError:
        return None
    return float(m.group(1)) if m else None


def build_model(w, device):
    import terapipe_amd as ta
    dt = TORCH_DTYPE[w["dtype"]]
    layers = ta.TransformerLayers(w["n_layers"], w["E"], w["F"], w["H"], dtype=dt, device=device)
    g = torch.Generator(device="cpu").manual_seed(0)
    with torch.no_grad():
        for p in layers.parameters():
            if p.dim() == 2:   # weights N(0, std); biases stay 0, LayerNorm gamma 1 / beta 0
                p.copy_((torch.randn(p.shape, generator=g) * w["std"]).to(dt))
    runner = ta.TeraPipe(layers, w["B"], w["L"], [w["B"]], w["slices"], slice_streams=1, launch_replay=False)
    x = torch.randn(w["L"], w["B"], w["E"], generator=g).to(dt).to(device)
    R = torch.randn(w["L"], w["B"], w["E"], generator=g).to(dt).to(device)
    return layers, runner, x, R


def one_step(layers, runner, x, R):
    for p in layers.parameters():
        p.grad = None
    y = runner(x)
    loss = (y * R).sum()
    loss.backward()
    return loss


def optimizer_step(layers, runner, x, R, reps=5):
    """update_weights of the reference's loop (16-bit gradients / 128 -> Adam on fp32 master weights -> 16-bit
    weights) as one tp_adam_step launch over every parameter of the stack, timed with HIP events.  HBM-bound:
    per parameter it reads 2 + 12 bytes and writes 12 + 2 (+ 2 for the zeroed gradient, kept here so that the
    launch can be repeated)."""
    import terapipe_amd as ta
    params = list(layers.parameters())
    master = [p.detach().clone().float() for p in params]
    opt = ta.FusedAdam(master, lr=1e-10)
    runner.use_hip_graph = False
    one_step(layers, runner, x, R)
    opt.update_weights(params, loss_scale=128.0, zero_grads=True)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        opt.update_weights(params, loss_scale=128.0, zero_grads=True)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / reps
    n = sum(p.numel() for p in params)
    nbytes = n * (2 + 12 + 12 + 2 + 2)
    return {"kernel": "tp::adam_kernel", "parameters": n, "tensors": len(params), "ms": ms, "bound": "hbm",
            "algorithmic_GB": nbytes / 1e9, "achieved_GBps": nbytes / (ms * 1e-3) / 1e9,
            "frac_of_hbm_peak": nbytes / (ms * 1e-3) / PEAK_HBM,
            "note": "includes the host's build and upload of the tensor table each call"}


def timed_steps(step, warmup, steps):
    """(ms per step, tokens-independent) of `step()` over `steps` calls after `warmup`, host clock between two
    synchronisations."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def layer_surface_step(layers, x, R, w, in_place=False, defer=False):
    """One step through the layer-level surface under the reference's own loop (terapipe.py:249-264 forward,
    :182-191 backward): per slice ``layers(x_i, cache, cache_len)`` with the caches detached and marked
    requires_grad, then in reverse ``autograd.backward([y_i] + cache_out_i, [dy_i] + da_{i+1})`` with
    ``da_i = cache_in_i.grad``.  Every slice is one autograd graph on the calling stream, one slice at a time --
    what a pipeline stage fed by an upstream stage runs."""
    import terapipe_amd as ta
    for p in layers.parameters():
        p.grad = None
    for layer in layers.layers:
        layer.accumulate_grads_in_place = in_place
        layer.defer_weight_grads = defer
    ss, B = w["slices"], w["B"]
    xs = ta.grid_slice_batch_and_sequence(x, [B], ss, requires_grad=True)
    dys = ta.grid_slice_batch_and_sequence(R, [B], ss)
    cache = layers.create_cache(B, w["L"])
    cin, cout, outs = [], [], []
    cache_len = 0
    for i, T in enumerate(ss):
        cache = [c.detach().requires_grad_() for c in cache]
        y, cache_out = layers(xs[0, i], cache, cache_len)
        cin.append(cache)
        cout.append(cache_out)
        outs.append(y)
        cache = cache_out
        cache_len += T
    da = []
    for i in reversed(range(len(ss))):
        a = list(cout[i]) if i < len(ss) - 1 else []
        torch.autograd.backward([outs[i]] + a, [dys[0, i]] + da)
        da = [t.grad for t in cin[i]]


def box_constants(device, dtype=torch.float16):
    """What this box delivers on two plain kernels, beside the published peaks the rooflines are priced against:
    a 1 GiB device-to-device copy (bytes read + written per second) and an 8192^3 product on N(0,1) operands (this
    library's tp_gemm and the vendor library behind torch.matmul), each replayed from a HIP graph between two events."""
    from terapipe_amd import ops, _lib
    n = 1 << 29
    src = torch.empty(n, dtype=torch.int16, device=device).random_(-9, 9)
    dst = torch.empty_like(src)
    ms = _graph_ms([lambda: dst.copy_(src)] * 4) / 4
    copy_gbps = 2 * n * 2 / (ms * 1e-3) / 1e9
    del src, dst
    M = 8192
    A = torch.randn(M, M, device=device).to(dtype)
    Bs = [torch.randn(M, M, device=device).to(dtype) for _ in range(3)]
    C = torch.empty(M, M, device=device, dtype=dtype)
    ours = _graph_ms([(lambda B=B: ops.gemm(_lib.TP_GEMM_NT, A, B, M, M, M, C=C)) for B in Bs]) / len(Bs)
    vend = _graph_ms([(lambda B=B: torch.matmul(A, B.t(), out=C)) for B in Bs]) / len(Bs)
    fl = 2.0 * M ** 3
    return {"copy_GBps": round(copy_gbps, 1), "copy_frac_of_hbm_peak": round(copy_gbps * 1e9 / PEAK_HBM, 4),
            "gemm_8192_TFLOPs": round(fl / (ours * 1e-3) / 1e12, 1),
            "gemm_8192_frac_of_mfma_peak": round(fl / (ours * 1e-3) / PEAK_MFMA_16BIT, 4),
            "vendor_gemm_8192_TFLOPs": round(fl / (vend * 1e-3) / 1e12, 1),
            "note": "measured on this box: 1 GiB device copy (read + write bytes); NT 8192^3 fp16 on N(0,1) operands, "
                    "tp_gemm and torch.matmul"}


def fill_path(device):
    """What the global -> LDS path delivers when nothing else runs (tp_fill_probe): every workgroup's four waves
    stream 8 KB batches into LDS, four batches in flight per wave and one 128 KB workgroup per CU -- the footprint
    of a GEMM tile ring -- from a 4 GiB region that no two waves share a byte of (HBM: misses) and / or a 2 MiB
    region (L2: hits), on 256, 128 and 64 CUs; a batch is 8 KB of consecutive bytes or a 64-row x 128-byte tile.  These rates bound every kernel here that stages operand tiles through LDS: a tile's bytes divided by the
    rate of its hit : miss mix is the least time a k-tile can take, whatever the MFMA pipe could do meanwhile."""
    from terapipe_amd import ops
    big = torch.empty(1 << 30, dtype=torch.int32, device=device).random_(0, 7)
    small = torch.empty(1 << 19, dtype=torch.int32, device=device).random_(0, 7)     # 2 MiB
    rows = []
    # consecutive bytes on 256, 128 and 64 CUs, then the tile walk of a GEMM's k loop (64 rows x 128 bytes, row pitch
    # 10240 bytes = a k of 5120 16-bit elements) on 256 CUs
    for wgs, stride in ((256, 0), (128, 0), (64, 0), (256, 10240)):
        for hpm, name in ((-1, "all L2 hits"), (7, "7 hits : 1 HBM"), (3, "3 : 1"), (1, "1 : 1"), (0, "all HBM")):
            batches = 512 if hpm != 0 else 256       # 256 workgroups x 4 waves x 512 batches x 8 KB = the 4 GiB
            nbytes = wgs * 4 * batches * 8192
            ms = _graph_ms([lambda: ops.fill_probe(big, small, hpm, wgs, batches, row_stride=stride)] * 3, 3) / 3
            rate = nbytes / (ms * 1e-3)
            hbm = rate * (0.0 if hpm < 0 else 1.0 / (hpm + 1))
            rows.append({"workgroups": wgs, "pattern": "consecutive bytes" if stride == 0 else "64 x 128 B tiles, row pitch %d B" % stride,
                         "mix": name, "us": round(ms * 1e3, 1), "GBps_per_CU": round(rate / wgs / 1e9, 1),
                         "chip_TBps": round(rate / 1e12, 2), "of_which_HBM_TBps": round(hbm / 1e12, 2)})
    return {"metric": "global -> LDS fill rate (global_load_lds_dwordx4, 128 KB of LDS and 16 batches of 8 KB in flight per CU)",
            "unit": "GB/s per CU, TB/s chip-wide", "peak_HBM_TBps": PEAK_HBM / 1e12, "rows": rows}


def in_step_picks():
    """{(op, M, N, K)} of the measured plan table's entries that were chosen by timing whole steps on the slice
    streams rather than the launch alone (their comments in gemm_tuned.inc say so): alone on the chip, as the
    per-GEMM roofline times them, they are not the fastest plan of their shape."""
    path = os.path.join(ROOT, "terapipe_amd", "csrc", "gemm_tuned.inc")
    ops_ = {"NT": 0, "NN": 1, "TN": 2}
    out = set()
    try:
        for line in open(path):
            m = re.match(r"\{TP_GEMM_(\w+), (\d+), (\d+), (\d+), (\d+), (\d+)\},\s*//(.*)", line)
            if m and ("in-step" in m.group(7) or "inside the step" in m.group(7)):
                out.add((ops_[m.group(1)], int(m.group(2)), int(m.group(3)), int(m.group(4))))
    except OSError:
        pass
    return out


def cpu_baseline(w, sample_layers=None):
    """The CPU oracle (fp32 restatement of the reference path) on this host's cores, on a bounded
    sample: the full sequence and slice list through `sample_layers` layers of the stack; the
    whole-stack rate is that rate divided by n_layers / sample_layers."""
    import oracle
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    flops_layer = gemm_flops_per_step(w) / w["n_layers"]
    sample_layers = sample_layers or max(1, min(w["n_layers"], int(1.3e13 // flops_layer)))
    ps = oracle.init_stack_params(sample_layers, w["E"], w["F"], w["std"], torch.float32, seed=0)
    for p in ps:
        for v in p.values():
            v.requires_grad_(True)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(w["L"], w["B"], w["E"], generator=g)
    R = torch.randn(w["L"], w["B"], w["E"], generator=g)
    t0 = time.time()
    oracle.terapipe_forward_backward(ps, x, R, w["H"], [w["B"]], w["slices"])
    dt = time.time() - t0
    tokens = w["L"] * w["B"]
    value = tokens / (dt * w["n_layers"] / sample_layers)
    return {"value": value, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": "fp32 torch-CPU oracle, full sequence and slice list through %d of %d layers, one step "
                      "(%.1f s), scaled by the layer count" % (sample_layers, w["n_layers"], dt)}


def vendor_gemm_us(metas, dtype, device):
    """{meta: microseconds} of torch.matmul on the products of each recorded GEMM call (a grouped call: its members
    one after the other), each alone on the chip, weights rotating over several buffers."""
    out = {}
    for meta in metas:
        members = meta if isinstance(meta[0], tuple) else (meta,)
        fns = []
        keep = []
        for (op, M, N, K) in members:
            nb = max(2, min(6, int(1.0e9 // (N * K * 2))))
            if op == 2:      # TN: C[M, N] = A[K, M]^T B[K, N]
                A = torch.randn(K, M, device=device, dtype=dtype)
                Bs = [torch.randn(K, N, device=device, dtype=dtype) for _ in range(2)]
                C = torch.empty(M, N, device=device, dtype=dtype)
                fns += [(lambda A=A, B=B, C=C: torch.matmul(A.t(), B, out=C)) for B in Bs]
            else:
                A = torch.randn(M, K, device=device, dtype=dtype)
                Bs = [torch.randn((N, K) if op == 0 else (K, N), device=device, dtype=dtype) for _ in range(nb)]
                C = torch.empty(M, N, device=device, dtype=dtype)
                fns += [(lambda A=A, B=B, C=C, op=op: torch.matmul(A, B.t() if op == 0 else B, out=C)) for B in Bs]
            keep.append((A, Bs, C))
        n_rounds = len(fns) // len(members) if len(members) > 1 else len(fns)
        out[meta] = _graph_ms(fns) * 1e3 / (n_rounds if len(members) == 1 else 2)
        del keep, fns
    return out


def _graph_ms(fns, reps=3):
    """Average milliseconds of one pass over `fns` (callables that launch on the current stream): the pass is
    captured into a HIP graph and the replays are bracketed by two HIP events on that stream, so no host
    launch gap is inside the figure."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for fn in fns[:4]:
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for fn in fns:
            fn()
    g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def measure_workload(name, args, device, detail):
    """Times `name`: tokens/s over args.steps steps after args.warmup, then (unless --no-roofline) the kernel
    times of one recorded step per kind.  detail: also per GEMM shape."""
    from terapipe_amd import ops
    w = WORKLOADS[name]
    args = argparse.Namespace(**vars(args))
    args.slice_streams = args.slice_streams or w.get("streams", 3)
    layers, runner, x, R = build_model(w, device)
    runner.use_hip_graph = args.graph
    runner.slice_streams = args.slice_streams
    runner.fused_attn_bwd = not args.two_launch_attn_bwd
    runner.launch_replay = not (args.graph or args.no_launch_replay)
    warmup, steps = (args.warmup, args.steps) if detail else (3, 5)
    for _ in range(warmup):
        one_step(layers, runner, x, R)
    torch.cuda.synchronize()
    # an event behind every step (recorded without waiting): the spread of the steps, as the reference's loop prints
    # mean and standard deviation (terapipe.py:290-315); the figure itself is the host clock around all K steps
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(steps):
        one_step(layers, runner, x, R)
        marks[i + 1].record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    per_step = [marks[i].elapsed_time(marks[i + 1]) for i in range(steps)]
    mean = sum(per_step) / steps
    res = {"workload": "%s: %s" % (name, w["desc"]), "dtype": w["dtype"], "steps": steps, "warmup": warmup,
           "ms_per_step": elapsed * 1e3 / steps, "tokens_per_s": w["L"] * w["B"] * steps / elapsed,
           "ms_per_step_std": (sum((t - mean) ** 2 for t in per_step) / steps) ** 0.5,
           "ms_per_step_min": min(per_step), "ms_per_step_max": max(per_step),
           "slice_streams": args.slice_streams}
    if args.slice_streams > 1 and not args.graph and not args.no_one_stream:
        # the same step with ONE slice stream: slice i+1 starts when slice i has left the stack, as on a pipeline
        # stage that receives its slices from an upstream stage (terapipe.py:249-264); recorded launches re-issued
        runner.slice_streams = 1
        ms1 = timed_steps(lambda: one_step(layers, runner, x, R), 3, 5)
        res["ms_per_step_one_stream"] = ms1
        res["tokens_per_s_one_stream"] = w["L"] * w["B"] / (ms1 * 1e-3)
        runner.slice_streams = args.slice_streams
    if detail and w["dtype"] != "f32" and not args.no_layer_surface:
        msl = timed_steps(lambda: layer_surface_step(layers, x, R, w), 2, 4)
        msi = timed_steps(lambda: layer_surface_step(layers, x, R, w, in_place=True), 2, 4)
        msd = timed_steps(lambda: layer_surface_step(layers, x, R, w, defer=True), 2, 4)
        for layer in layers.layers:
            layer.accumulate_grads_in_place = layer.defer_weight_grads = False
        res["layer_surface"] = {
            "ms_per_step": msl, "tokens_per_s": w["L"] * w["B"] / (msl * 1e-3),
            "ms_per_step_grads_in_place": msi, "tokens_per_s_grads_in_place": w["L"] * w["B"] / (msi * 1e-3),
            "ms_per_step_deferred_weight_grads": msd,
            "tokens_per_s_deferred_weight_grads": w["L"] * w["B"] / (msd * 1e-3),
            "what": "ModelParallelTransformerLayer.forward per slice under the reference's own loop and autograd "
                    "(terapipe.py:249-264, :182-191): per-slice parameter-gradient GEMMs, gradient caches, one stream, "
                    "every launch issued from Python; grads_in_place: with accumulate_grads_in_place=True, the "
                    "slices after the first add their parameter gradients to .grad inside the gradient kernels; "
                    "deferred_weight_grads: with defer_weight_grads=True, a sequence's weight gradients are taken once, "
                    "in the backward of its first slice, over all its rows"}
    if args.no_roofline:
        return res, (layers, runner, x, R)

    # Kernel time per kind, measured live with HIP events: one step is recorded (every library call
    # with its descriptor and buffers), then all calls of one kind are replayed back to back inside
    # a HIP graph on the launch stream and the replay is bracketed by two events.  Replaying from a
    # graph keeps host launch gaps out of the figure (events around single eager launches would
    # include the time the GPU waits for the host).
    runner.use_hip_graph = False
    runner.launch_replay = False
    with ops.CallRecorder() as rec:
        one_step(layers, runner, x, R)
    torch.cuda.synchronize()
    # the recorded weight-gradient GEMMs write into this step's gradient tensors: keep them alive while
    # the calls are replayed
    recorded_grads = [p.grad for p in layers.parameters()]
    es = 4 if w["dtype"] == "f32" else 2
    peak = PEAK_MFMA_FP32 if w["dtype"] == "f32" else PEAK_MFMA_16BIT

    def calls_of(tag):
        # "attn_bwd" covers both launches of the attention backward of a slice: delta + dQ, and the
        # one-pass dK/dV over all later positions
        return [c for c in rec.calls if c[0] == tag or (tag == "attn_bwd" and c[0] == "attn_bwd_dkdv")]

    gemm_calls = calls_of("gemm")
    g_ms = _graph_ms([fn for _, _, fn in gemm_calls])
    flops = gemm_flops_per_step(w)
    achieved = flops / (g_ms * 1e-3)
    # what the rooflines allow each launch: the larger of its MFMA time and the time to move its operands
    # and result through HBM once
    work = [gemm_shape_work(m, es) for _, m, _ in gemm_calls]
    bound_s = sum(max(f / peak, b / PEAK_HBM) for f, b in work)
    attainable = sum(f for f, _ in work) / bound_s
    roof = {
        "kernel": "tp::gemm_pipe_kernel / tp::gemm_tall_kernel / tp::gemm_dma_kernel / tp::gemm_stream_kernel (all NT/NN/TN launches of one step, "
                  "split-K reduce included)",
        "bound": "mfma", "achieved": achieved / 1e12, "peak": peak / 1e12, "unit": "TFLOP/s",
        "frac": achieved / peak, "traffic": pmc_traffic(name),
        "traffic_note": "bytes per launch that L2 exchanges with the fabric (the memory-side cache serves part of them): rocprofv3 "
                        "FETCH_SIZE / 0.500 + WRITE_SIZE / 1.000, the factors read off a plain copy and a fill of known size in "
                        "the same counter runs; from the committed profiles/ summary of one eager step",
        "algorithmic_bytes_per_launch": sum(b for _f, b in work) / max(len(gemm_calls), 1),
        "launches": len(gemm_calls), "avg_launch_us": g_ms * 1e3 / max(len(gemm_calls), 1),
        "algorithmic_flops_per_step": flops, "kernel_ms_per_step": g_ms,
        "attainable": attainable / 1e12, "attainable_frac": attainable / peak,
        "achieved_over_attainable": achieved / attainable,
        "attainable_note": "per launch min(MFMA peak, (A + B + C bytes) / 8 TB/s), summed over the step's launches",
        "method": "graph replay of the step's GEMM calls between two HIP events, one after the other on one stream: each "
                  "launch has the chip to itself, with the tile and k splits the step uses (several of those were "
                  "chosen by timing whole steps on the slice streams and are not the fastest alone; shared_chip times "
                  "the same launches as the step overlaps them)",
    }
    if detail:
        groups = {}
        for c in gemm_calls:
            groups.setdefault(c[1], []).append(c[2])
        groups = dict(sorted(groups.items(), key=lambda kv: str(kv[0])))
        per = []
        picks = in_step_picks()
        for meta, fns in groups.items():
            ms = _graph_ms(fns)
            f, b = gemm_shape_work(meta, es)
            us = ms * 1e3 / len(fns)
            bound_us = max(f / peak, b / PEAK_HBM) * 1e6
            per.append({"gemm": gemm_shape_name(meta), "calls": len(fns), "avg_us": round(us, 2),
                        "tflops": round(f / us / 1e6, 1), "bound_us": round(bound_us, 2),
                        "bound": "mfma" if f / peak >= b / PEAK_HBM else "hbm",
                        "frac_of_bound": round(bound_us / us, 3),
                        # the plan of this shape was chosen by timing whole steps, not this launch alone
                        "in_step_pick": (not isinstance(meta[0], tuple)) and tuple(meta) in picks})
        if not args.no_vendor_gemm:
            # context only: the vendor library (hipBLASLt / rocBLAS behind torch.matmul) on the same products, plain
            # (no fused epilogue), timed the same way over weights that rotate through more memory than the caches hold
            vend = vendor_gemm_us(list(groups), TORCH_DTYPE[w["dtype"]], device)
            vt = 0.0
            for r, meta in zip(per, groups):
                r["vendor_us"] = round(vend[meta], 2)
                vt += vend[meta] * r["calls"]
            roof["vendor_library"] = {"kernel_ms_per_step": vt * 1e-3, "achieved": flops / (vt * 1e-6) / 1e12,
                                      "frac": flops / (vt * 1e-6) / peak,
                                      "note": "torch.matmul on the same (op, M, N, K) list, plain products, context only"}
        per.sort(key=lambda r: -r["avg_us"] * r["calls"])
        roof["per_gemm"] = per
        roof["per_gemm_note"] = ("avg_us is the launch alone on the chip with the plan the step uses; in_step_pick marks "
                                 "the shapes whose plan was chosen by timing whole steps on the slice streams (fewer k "
                                 "splits than the fastest plan alone), so vendor_us may be below avg_us there")
    if args.slice_streams > 1:
        # the same GEMM calls as the step issues them: spread over the slice streams, so that a launch
        # which fills part of the chip runs beside its neighbours'.  Launched from the host (closures
        # bound to their descriptors), bracketed by two events on the current stream.  Every chain has a
        # k-split workspace of its own, as the runner's streams have.
        chains = [torch.cuda.Stream() for _ in range(args.slice_streams)]
        ws_bytes = max([b.numel() for b in ops.Workspace._bufs.values()] + [1 << 20])
        chain_ws = [torch.empty(ws_bytes, dtype=torch.uint8, device=device) for _ in chains]
        main = torch.cuda.current_stream()

        def spread():
            for st in chains:
                st.wait_stream(main)
            for i, (_, _, fn) in enumerate(gemm_calls):
                k = i % len(chains)
                if fn(chains[k].cuda_stream, ws=chain_ws[k]):
                    raise RuntimeError("replayed GEMM failed")
            for st in chains:
                main.wait_stream(st)
        spread()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(3):
            spread()
        e1.record()
        torch.cuda.synchronize()
        c_ms = e0.elapsed_time(e1) / 3
        roof["shared_chip"] = {
            "chains": len(chains), "kernel_ms_per_step": c_ms, "achieved": flops / (c_ms * 1e-3) / 1e12,
            "frac": flops / (c_ms * 1e-3) / peak,
            "method": "the step's GEMM calls issued round-robin over the slice streams, as the step overlaps them"}
        del chain_ws
    res["roofline"] = roof
    attn = {}
    kt = {"gemm": round(g_ms, 3)}
    has_suffix = any(c[0] == "attn_bwd_dkdv" for c in rec.calls)
    for tag in ("attn_fwd", "attn_bwd"):
        calls = calls_of(tag)
        ms = _graph_ms([fn for _, _, fn in calls]) if calls else 0.0
        metas = [m for t, m, _ in calls if t == tag]     # one per slice and layer
        nbytes = sum(attn_bytes_per_call(es, w["B"], w["H"], w["E"], T, P, tag == "attn_bwd") for (_b, _h, _d, T, P) in metas)
        gbs = nbytes / (ms * 1e-3) / 1e9 if ms > 0 else 0.0
        attn[tag] = {"calls": len(metas), "launches_per_call": 2 if tag == "attn_bwd" and has_suffix else 1,
                     "kernel_ms_per_step": ms, "algorithmic_GB_per_step": nbytes / 1e9,
                     "achieved_GBps": gbs, "frac_of_hbm_peak": gbs * 1e9 / PEAK_HBM}
        kt[tag] = round(ms, 3)
    for tag in ("layernorm_fwd", "layernorm_bwd"):
        calls = calls_of(tag)
        kt[tag] = round(_graph_ms([fn for _, _, fn in calls]) if calls else 0.0, 3)
    res["roofline_attention"] = {"bound": "hbm", "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                                 "slice_tokens": sorted(set(w["slices"])), **attn}
    res["kernel_time_ms_per_step"] = kt
    del recorded_grads
    return res, (layers, runner, x, R)


def attention_grid(device, reps=5):
    """The (T, P) micro-grid of the prefix-attention kernels, as the reference profiles a layer per
    (seqlen, attention_cache_len) (terapipe_latency_model.py:180-193): slice length T in {32, 64, 128}, prefix P
    in {0, 256, ..., 1792, 2048 - T} of a 2048-token sequence, head dimension 128, bf16, at the (batch, heads) of
    workloads C5 (2, 48) and C4 (1, 96).  Per point: the forward call; the backward as the sliced runner issues
    it -- ONE launch for the slice at P whose first half takes delta + dQ against the P keys before the slice and
    whose second half takes dK/dV of the slice's keys over the L - P queries from the slice on, with the delta of three
    slices' positions taken inside the launch as the three-stream runner has it (bwd_fused_us; its
    two halves as separate launches: dq_us at P, and dkdv_mirror_us = the dK/dV launch of the slice at the mirrored
    position L - T - P, which covers as many query-key blocks as dQ at P does); and the backward with gradient
    caches (the reference's per-call contract: dK/dV of all S keys, prefix rows read-modify-written).  The fused
    launch does a whole row AND a whole column of the causal triangle per slice, so its time hardly depends on P;
    "sequence" sums bytes and times over the grid's positions, which is what a step over the whole sequence sees.  Each call is timed alone on the chip over `sets` rotating sets of buffers larger
    together than the memory-side cache, replayed from a HIP graph between two HIP events; GB/s are the
    reference algorithm's bytes of the call (fwd (2T+2S) B E, bwd (6T+2S+4P) B E, + fp32 row statistics)."""
    from terapipe_amd import ops
    L, Dh, dt, es = 2048, 128, torch.bfloat16, 2
    out = []
    for wl, (B, H) in (("C5", (2, 48)), ("C4", (1, 96))):
        BH, E = B * H, H * Dh
        sets = 6
        g = torch.Generator(device=device).manual_seed(7)
        bufs = []
        for _ in range(sets):
            b = dict(q=torch.randn(BH, L, Dh, generator=g, device=device).to(dt) * Dh ** -0.5,
                     k=torch.randn(BH, L, Dh, generator=g, device=device).to(dt),
                     v=torch.randn(BH, L, Dh, generator=g, device=device).to(dt),
                     o=torch.empty(L, B, E, dtype=dt, device=device),
                     d_o=torch.randn(L, B, E, generator=g, device=device).to(dt),
                     lse=torch.zeros(BH, L, dtype=torch.float32, device=device),
                     delta=torch.zeros(BH, L, dtype=torch.float32, device=device),
                     dqkv=torch.empty(128 * B, 3 * E, dtype=dt, device=device),
                     gk=torch.zeros(BH, L, Dh, dtype=torch.float32, device=device),
                     gv=torch.zeros(BH, L, Dh, dtype=torch.float32, device=device))
            bufs.append(b)
        # every position's lse / delta / o must be valid for the one-pass dK/dV: one forward + dQ sweep first
        for b in bufs:
            for P in range(0, L, 128):
                ops.attn_prefix_fwd(b["q"][:, P:], b["k"], b["v"], B, H, Dh, 128, P, Dh ** -0.5, out=b["o"][P:P + 128],
                                    lse=b["lse"][:, P:], q_bh_rows=L, stat_bh_rows=L)
                ops.attn_prefix_bwd(b["q"][:, P:], b["k"], b["v"], b["o"][P:P + 128], b["lse"][:, P:], b["d_o"][P:P + 128],
                                    b["dqkv"], None, None, B, H, Dh, 128, P, Dh ** -0.5, False, False, False,
                                    delta=b["delta"][:, P:], q_bh_rows=L, stat_bh_rows=L, dq_only=True)
        torch.cuda.synchronize()
        for T in (32, 64, 128):
            rows = []
            for P in sorted(set(list(range(0, L - T, 256)) + [L - T])):
                def fwd(b, T=T, P=P):
                    ops.attn_prefix_fwd(b["q"][:, P:], b["k"], b["v"], B, H, Dh, T, P, Dh ** -0.5, out=b["o"][P:P + T],
                                        lse=b["lse"][:, P:], q_bh_rows=L, stat_bh_rows=L)

                def dq(b, T=T, P=P):
                    ops.attn_prefix_bwd(b["q"][:, P:], b["k"], b["v"], b["o"][P:P + T], b["lse"][:, P:], b["d_o"][P:P + T],
                                        b["dqkv"][:T * B], None, None, B, H, Dh, T, P, Dh ** -0.5, False, False, False,
                                        delta=b["delta"][:, P:], q_bh_rows=L, stat_bh_rows=L, dq_only=True)

                def dkdv(b, T=T, P=P):
                    # the one-pass dK/dV of the slice at the mirrored position L - T - P: it visits as many (query,
                    # key) blocks as this slice has prefix + diagonal blocks, so over a whole sequence of T-token
                    # slices the pairs (dQ at P, dK/dV at L - T - P) are exactly the backward launches of a step
                    ops.attn_suffix_dkdv(b["k"], b["v"], b["q"], b["d_o"], b["lse"], b["delta"], b["dqkv"][:T * B], B, H, Dh,
                                         L - T - P, T, L)

                def fused(b, T=T, P=P):
                    ops.attn_bwd_fused(b["q"][:, P:], b["k"], b["v"], b["o"][P:P + T], b["lse"][:, P:], b["d_o"][P:P + T],
                                       b["dqkv"][:T * B], B, H, Dh, T, P, Dh ** -0.5, b["delta"][:, P:], b["q"], b["d_o"],
                                       b["lse"], b["delta"], b["o"], L, own_delta_end=min(L, P + 3 * T), q_bh_rows=L,
                                       stat_bh_rows=L)

                def bwd_cache(b, T=T, P=P):
                    ops.attn_prefix_bwd(b["q"][:, P:], b["k"], b["v"], b["o"][P:P + T], b["lse"][:, P:], b["d_o"][P:P + T],
                                        b["dqkv"][:T * B], b["gk"], b["gv"], B, H, Dh, T, P, Dh ** -0.5, True, True, False,
                                        delta=b["delta"][:, P:], q_bh_rows=L, stat_bh_rows=L)

                us = {}
                for nm, fn in (("fwd", fwd), ("dq", dq), ("dkdv", dkdv), ("fused", fused), ("bwd_cache", bwd_cache)):
                    us[nm] = _graph_ms([(lambda b=b, fn=fn: fn(b)) for b in bufs], reps) * 1e3 / sets
                fb = attn_bytes_per_call(es, B, H, E, T, P, False)
                bb = attn_bytes_per_call(es, B, H, E, T, P, True)
                run_us = us["dq"] + us["dkdv"]
                rows.append({"P": P, "fwd_us": round(us["fwd"], 2), "fwd_GBps": round(fb / us["fwd"] / 1e3, 1),
                             "dq_us": round(us["dq"], 2), "dkdv_mirror_us": round(us["dkdv"], 2),
                             "bwd_two_launches_us": round(run_us, 2), "bwd_two_launches_GBps": round(bb / run_us / 1e3, 1),
                             "bwd_fused_us": round(us["fused"], 2),
                             "bwd_cache_us": round(us["bwd_cache"], 2), "bwd_cache_GBps": round(bb / us["bwd_cache"] / 1e3, 1),
                             "fwd_bytes": fb, "bwd_bytes": bb})
            seq = {}
            for nm, ub, uk in (("fwd", "fwd_bytes", "fwd_us"), ("bwd_fused", "bwd_bytes", "bwd_fused_us"),
                               ("bwd_two_launches", "bwd_bytes", "bwd_two_launches_us"), ("bwd_cache", "bwd_bytes", "bwd_cache_us")):
                gbs = sum(r[ub] for r in rows) / sum(r[uk] for r in rows) / 1e3
                seq[nm + "_GBps"] = round(gbs, 1)
                seq[nm + "_frac_of_hbm_peak"] = round(gbs * 1e9 / PEAK_HBM, 4)
            out.append({"heads_of": wl, "batch": B, "heads": H, "T": T, "sequence": seq, "points": rows})
        del bufs
        gc.collect()
        torch.cuda.empty_cache()
    return {"metric": "prefix-attention kernel time and achieved HBM GB/s per (T, P)", "unit": "us, GB/s",
            "dtype": "bf16", "head_dim": Dh, "seq": L, "peak_GBps": PEAK_HBM / 1e9,
            "method": "each call alone on the chip over 6 rotating buffer sets, HIP-graph replay between two HIP events",
            "grid": out}


def _short(res):
    """The other workloads' figures in short."""
    s = {"workload": res["workload"], "ms_per_step": round(res["ms_per_step"], 3),
         "tokens_per_s": round(res["tokens_per_s"], 1), "slice_streams": res["slice_streams"]}
    if "ms_per_step_one_stream" in res:
        s["ms_per_step_one_stream"] = round(res["ms_per_step_one_stream"], 3)
        s["tokens_per_s_one_stream"] = round(res["tokens_per_s_one_stream"], 1)
    if "roofline" in res:
        r = res["roofline"]
        s["gemm"] = {"kernel_ms_per_step": round(r["kernel_ms_per_step"], 3), "achieved_TFLOPs": round(r["achieved"], 1),
                     "frac": round(r["frac"], 4), "attainable_frac": round(r["attainable_frac"], 4)}
        if "shared_chip" in r:
            s["gemm"]["shared_chip_frac"] = round(r["shared_chip"]["frac"], 4)
        a = res["roofline_attention"]
        s["attention"] = {k: {"kernel_ms_per_step": round(a[k]["kernel_ms_per_step"], 3),
                              "achieved_GBps": round(a[k]["achieved_GBps"], 1),
                              "frac_of_hbm_peak": round(a[k]["frac_of_hbm_peak"], 4)} for k in ("attn_fwd", "attn_bwd")}
        s["kernel_time_ms_per_step"] = res["kernel_time_ms_per_step"]
    return s


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="C3", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-roofline", action="store_true")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="with the default workload C3 the line also carries the prefix-attention roofline measured on C5 "
                         "(32-token slices) and short figures for C2, C4 and C5; this leaves them out")
    ap.add_argument("--no-one-stream", action="store_true",
                    help="leave out the timing of the same step on one slice stream")
    ap.add_argument("--no-layer-surface", action="store_true",
                    help="leave out the timing of the layer-level surface under the reference's own slice loop")
    ap.add_argument("--layer-surface-only", action="store_true",
                    help="time only the layer-level surface (the reference's per-slice loop under autograd) for "
                         "--steps steps after --warmup and print its line: the run to put under a kernel trace")
    ap.add_argument("--grads-in-place", action="store_true",
                    help="with --layer-surface-only: set accumulate_grads_in_place on the layers")
    ap.add_argument("--defer-weight-grads", action="store_true",
                    help="with --layer-surface-only: set defer_weight_grads on the layers")
    ap.add_argument("--no-box-constants", action="store_true",
                    help="leave out the measured copy bandwidth and 8192^3 GEMM rate of this box")
    ap.add_argument("--no-vendor-gemm", action="store_true",
                    help="leave out the vendor library's times on the same GEMM shapes (context beside the per-GEMM table)")
    ap.add_argument("--attention-grid", action="store_true",
                    help="print the (T, P) micro-grid of the prefix-attention kernels instead of the step benchmark")
    ap.add_argument("--fill-path", action="store_true",
                    help="print what the global -> LDS path of the CUs delivers (hits, misses and mixes) instead of the "
                         "step benchmark")
    ap.add_argument("--two-launch-attn-bwd", action="store_true",
                    help="issue dQ and the one-pass dK/dV of a slice as two launches instead of one (comparison)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 256 MiB device fill and one 256 MiB copy before the steps: the "
                         "known-size kernels that rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings are scaled by")
    ap.add_argument("--slice-streams", type=int, default=None,
                    help="streams the runner spreads consecutive slices over (default: the workload's own, 3 except "
                         "C2's 4; 1 = one chain of kernels); slice "
                         "i+1 of layer l runs beside slice i of layer l+1, which fills the CUs the short kernels "
                         "of one slice leave idle")
    ap.add_argument("--optimizer", action="store_true",
                    help="also time the mixed-precision Adam update (fp32 master weights, loss scale 128) that "
                         "follows the step in the reference's training loop; reported beside, never inside, value")
    ap.add_argument("--graph", action="store_true",
                    help="replay the runner's HIP graphs (forward, backward) instead of launching every kernel "
                         "from the host each step; one stream only")
    ap.add_argument("--eager", action="store_true", help="launch every kernel from the host (the default)")
    ap.add_argument("--no-launch-replay", action="store_true",
                    help="rebuild every descriptor in Python each step instead of re-issuing the launches recorded "
                         "on the second step")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path is built and measured on ONE GPU; --gpus %d is not supported "
              "(no collectives or sharding are part of this build)" % args.gpus, file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.attention_grid:
        print(json.dumps(attention_grid(device)))
        return
    if args.fill_path:
        print(json.dumps(fill_path(device)))
        return
    if args.slice_streams is not None and args.slice_streams < 1:
        print("bench.py: --slice-streams must be at least 1", file=sys.stderr)
        sys.exit(2)
    if args.graph and (args.eager or args.slice_streams != 1):
        print("bench.py: --graph replays a single-stream capture; use it with --slice-streams 1 and without --eager",
              file=sys.stderr)
        sys.exit(2)
    w = WORKLOADS[args.workload]
    if args.layer_surface_only:
        layers, runner, x, R = build_model(w, device)
        del runner
        ms = timed_steps(lambda: layer_surface_step(layers, x, R, w, args.grads_in_place, args.defer_weight_grads),
                         args.warmup, args.steps)
        print(json.dumps({"workload": "%s: %s" % (args.workload, w["desc"]), "layer_surface_ms_per_step": ms,
                          "accumulate_grads_in_place": args.grads_in_place,
                          "defer_weight_grads": args.defer_weight_grads,
                          "tokens_per_s": w["L"] * w["B"] / (ms * 1e-3), "steps": args.steps, "warmup": args.warmup}))
        return
    if args.copy_calibration:
        src = torch.ones(64 << 20, dtype=torch.int32, device=device)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    res, model = measure_workload(args.workload, args, device, detail=True)
    out = {
        "metric": "sliced-layer fwd+bwd tokens/s on 1 MI355X; % MFMA peak (GEMM), % HBM BW (attn)",
        "value": res["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": res["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "ms_per_step_std": res["ms_per_step_std"], "ms_per_step_min": res["ms_per_step_min"],
        "ms_per_step_max": res["ms_per_step_max"],
        "dtype": w["dtype"], "data": "synthetic",
        "config": {"workload": res["workload"],
                   "loss": "sum(y * R), R ~ N(0,1) fixed", "optimizer_step": "outside the timed step (--optimizer times it separately)",
                   "launch": "HIP-graph replay of forward and of backward" if args.graph else
                             ("eager, every kernel launched from the host" if args.no_launch_replay else
                              "eager, recorded launches re-issued from the host"),
                   "slice_streams": res["slice_streams"]},
    }
    for k in ("ms_per_step_one_stream", "tokens_per_s_one_stream", "layer_surface", "roofline", "kernel_time_ms_per_step"):
        if k in res:
            out[k] = res[k]
    if "ms_per_step_one_stream" in res:
        out["one_stream_note"] = ("value / ms_per_step overlap three consecutive slices on three streams of the one GPU; "
                                  "*_one_stream run one slice at a time, as a pipeline stage fed by an upstream stage does")
    if "roofline_attention" in res:
        out["roofline_attention"] = dict(res["roofline_attention"], workload=args.workload)
    if args.optimizer and w["dtype"] != "f32":
        out["optimizer_step"] = optimizer_step(*model)
    del model
    gc.collect()
    torch.cuda.empty_cache()

    if args.workload == "C3" and not args.no_other_workloads and not args.no_roofline:
        # the prefix-attention target is stated for slices of at most 128 tokens: C5 (32-token slices) gives the
        # line's roofline_attention, the 13B workload's own attention figures move to roofline_attention_C3
        others = {}
        for name in ("C5", "C4", "C2"):
            r, m = measure_workload(name, args, device, detail=False)
            del m
            gc.collect()
            torch.cuda.empty_cache()
            others[name] = _short(r)
            if name == "C5":
                out["roofline_attention_C3"] = out["roofline_attention"]
                out["roofline_attention"] = dict(r["roofline_attention"], workload="C5")
        out["other_workloads"] = others

    if not args.no_box_constants and w["dtype"] != "f32":
        out["box"] = box_constants(device, TORCH_DTYPE[w["dtype"]])
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w)

    print(json.dumps(out))


if __name__ == "__main__":
    main()
