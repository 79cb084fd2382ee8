#!/usr/bin/env python3
"""Headline benchmark: sliced GPT-layer-stack forward + reverse-slice backward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C2|C3|C4|C5|C1]

One step = every sequence slice of one synthetic batch through the whole layer stack forward (K/V
caches growing slice by slice), then the reverse-order slice backward, with the loss
``sum(y * R)`` for a fixed random R (inputs N(0,1), weights N(0,0.02), all resident in HBM before the
timed region).  Prints ONE JSON line: tokens/s, the MFMA roofline of the GEMM kernels (algorithmic
flops / kernel time, measured live: the GEMM calls of one recorded step replayed in a HIP graph between
two HIP events), the HBM figure of the prefix-attention kernels, and the CPU oracle timed on this host's cores on a bounded sample.
"""
import argparse
import json
import os
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

# HBM bytes per GEMM call (FETCH_SIZE + WRITE_SIZE of the GEMM kernels of one step / calls), from the two
# rocprofv3 --pmc runs summarised in profiles/bench_C2_gemm_hbm_traffic.pmc.txt; only measured for C2
PMC_GEMM_TRAFFIC_BYTES = {"C2": 32.86e6}

WORKLOADS = {
    # name: layers, hidden, heads, ffn, seq, batch, dtype, slices, weight std
    "C1": dict(desc="tiny GPT stack fp32: 4 layers, hidden 256, 4 heads, FFN 1024, seq 128, batch 2, 8x16 slices",
               n_layers=4, E=256, H=4, F=1024, L=128, B=2, dtype="f32", slices=[16] * 8, std=0.02),
    "C2": dict(desc="GPT-3 1.3B shape: 24 layers, hidden 2048, 16 heads, FFN 8192, seq 2048, batch 1, fp16, 8x256 slices",
               n_layers=24, E=2048, H=16, F=8192, L=2048, B=1, dtype="f16", slices=[256] * 8, std=0.02),
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


def gemm_flops_per_step(w):
    """72 * E^2 flops per token per layer fwd+bwd for F = 4E; stated generally as
    3 passes (fwd, dX, dW) x 2 * (3E*E + E*E + 2*E*F) per token."""
    per_token_fwd = 2 * (3 * w["E"] * w["E"] + w["E"] * w["E"] + 2 * w["E"] * w["F"])
    return 3 * per_token_fwd * w["L"] * w["B"] * w["n_layers"]


def attn_bytes_per_call(w, T, P, bwd):
    """Algorithmic HBM bytes of one prefix-attention call (one layer, one slice): elements x dtype size
    plus the fp32 LSE / delta vectors.  fwd (2T + 2S) B E; bwd (6T + 2S + 4P) B E."""
    es = 4 if w["dtype"] == "f32" else 2
    S, BE, BH = P + T, w["B"] * w["E"], w["B"] * w["H"]
    if not bwd:
        return (2 * T + 2 * S) * BE * es + 4 * BH * T
    return (6 * T + 2 * S + 4 * P) * BE * es + 8 * BH * T


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


def cpu_baseline(w, budget_layers=None):
    """The CPU oracle (fp32 restatement of the reference path) on this host's cores, on a bounded
    sample: the full sequence and slice list through `sample_layers` layers of the stack; the
    whole-stack rate is that rate divided by n_layers / sample_layers."""
    import oracle
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    flops_layer = gemm_flops_per_step(w) / w["n_layers"]
    sample_layers = budget_layers or max(1, min(w["n_layers"], int(1.5e13 // flops_layer)))
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="C2", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-roofline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 256 MiB device copy (torch copy_ kernel) before the steps: the "
                         "known-size kernel that rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings are scaled by")
    ap.add_argument("--slice-streams", type=int, default=3,
                    help="streams the runner spreads consecutive slices over (1 = one chain of kernels); slice "
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
    w = WORKLOADS[args.workload]
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    from terapipe_amd import ops

    layers, runner, x, R = build_model(w, device)
    if args.graph and (args.eager or args.slice_streams != 1):
        print("bench.py: --graph replays a single-stream capture; use it with --slice-streams 1 and without --eager",
              file=sys.stderr)
        sys.exit(2)
    runner.use_hip_graph = args.graph
    runner.slice_streams = args.slice_streams
    runner.launch_replay = not (args.graph or args.no_launch_replay)
    if args.copy_calibration:
        src = torch.ones(64 << 20, dtype=torch.int32, device=device)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        one_step(layers, runner, x, R)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        one_step(layers, runner, x, R)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    tokens = w["L"] * w["B"]
    value = tokens * args.steps / elapsed

    out = {
        "metric": "sliced-layer fwd+bwd tokens/s on 1 MI355X; % MFMA peak (GEMM), % HBM BW (attn)",
        "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w["dtype"], "data": "synthetic",
        "config": {"workload": "%s: %s" % (args.workload, w["desc"]),
                   "loss": "sum(y * R), R ~ N(0,1) fixed", "optimizer_step": "outside the timed step (--optimizer times it separately)",
                   "launch": "HIP-graph replay of forward and of backward" if args.graph else
                             ("eager, every kernel launched from the host" if args.no_launch_replay else
                              "eager, recorded launches re-issued from the host"),
                   "slice_streams": args.slice_streams},
    }

    if not args.no_roofline:
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

        def replay_ms(tag, reps=3):
            # "attn_bwd" covers both launches of the attention backward of a slice: delta + dQ, and the
            # one-pass dK/dV over all later positions
            calls = [c for c in rec.calls if c[0] == tag or (tag == "attn_bwd" and c[0] == "attn_bwd_dkdv")]
            if not calls:
                return 0, 0.0, []
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _, _, fn in calls[:4]:
                    fn()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                for _, _, fn in calls:
                    fn()
            g.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                g.replay()
            e1.record()
            torch.cuda.synchronize()
            return len(calls), e0.elapsed_time(e1) / reps, [m for _, m, _ in calls]

        g_calls, g_ms, _ = replay_ms("gemm")
        flops = gemm_flops_per_step(w)
        peak = PEAK_MFMA_FP32 if w["dtype"] == "f32" else PEAK_MFMA_16BIT
        achieved = flops / (g_ms * 1e-3) if g_ms > 0 else 0.0
        out["roofline"] = {
            "kernel": "tp::gemm_dma_kernel / tp::gemm_tall_kernel (all NT/NN/TN launches of one step, split-K reduce included)",
            "bound": "mfma", "achieved": achieved / 1e12, "peak": peak / 1e12, "unit": "TFLOP/s",
            "frac": achieved / peak, "traffic": PMC_GEMM_TRAFFIC_BYTES.get(args.workload),
            "launches": g_calls, "avg_launch_us": g_ms * 1e3 / max(g_calls, 1),
            "algorithmic_flops_per_step": flops, "kernel_ms_per_step": g_ms,
            "method": "graph replay of the step's GEMM calls between two HIP events",
        }
        if args.slice_streams > 1:
            # the same GEMM calls as the step issues them: spread over the slice streams, so that a launch
            # which fills part of the chip runs beside its neighbours'.  Launched from the host (closures
            # bound to their descriptors), bracketed by two events on the current stream.
            chains = [torch.cuda.Stream() for _ in range(args.slice_streams)]
            calls = [c for c in rec.calls if c[0] == "gemm"]
            main = torch.cuda.current_stream()

            def spread():
                for st in chains:
                    st.wait_stream(main)
                for i, (_, _, fn) in enumerate(calls):
                    if fn(chains[i % len(chains)].cuda_stream):
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
            out["roofline"]["shared_chip"] = {
                "chains": len(chains), "kernel_ms_per_step": c_ms, "achieved": flops / (c_ms * 1e-3) / 1e12,
                "frac": flops / (c_ms * 1e-3) / peak,
                "method": "the step's GEMM calls issued round-robin over the slice streams, as the step overlaps them"}
        attn = {}
        kt = {"gemm": round(g_ms, 3)}
        for tag in ("attn_fwd", "attn_bwd"):
            c, ms, metas = replay_ms(tag)
            nbytes = sum(attn_bytes_per_call(w, T, P, tag == "attn_bwd") for (_b, _h, _d, T, P) in metas) / \
                (2 if tag == "attn_bwd" and any(c[0] == "attn_bwd_dkdv" for c in rec.calls) else 1)
            gbs = nbytes / (ms * 1e-3) / 1e9 if ms > 0 else 0.0
            if tag == "attn_bwd" and any(cc[0] == "attn_bwd_dkdv" for cc in rec.calls):
                c //= 2      # two library calls per slice backward
            attn[tag] = {"calls": c, "kernel_ms_per_step": ms, "algorithmic_GB_per_step": nbytes / 1e9,
                         "achieved_GBps": gbs, "frac_of_hbm_peak": gbs * 1e9 / PEAK_HBM}
            kt[tag] = round(ms, 3)
        for tag in ("layernorm_fwd", "layernorm_bwd"):
            kt[tag] = round(replay_ms(tag)[1], 3)
        out["roofline_attention"] = {"bound": "hbm", "peak": PEAK_HBM / 1e9, "unit": "GB/s", **attn}
        out["kernel_time_ms_per_step"] = kt

        del recorded_grads

    if args.optimizer and w["dtype"] != "f32":
        out["optimizer_step"] = optimizer_step(layers, runner, x, R)

    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w)

    print(json.dumps(out))


if __name__ == "__main__":
    main()
