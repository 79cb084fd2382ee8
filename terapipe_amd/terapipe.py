"""Host-side mirror of the reference's sliced runner (terapipe.py of the reference) on one GPU:
``TransformerLayers`` (terapipe.py:52-95) and ``TeraPipe`` (terapipe.py:219-271) with the reverse-order
slice backward of ``TeraPipeBackwardPassHook`` (terapipe.py:154-212).

``TeraPipe.forward`` runs the whole slice grid inside ONE autograd node on buffers allocated once per
runner.  Its backward walks the slices in reverse, hands dK/dV of the prefix rows from slice i+1 to
slice i through persistent fp32 gradient caches (instead of a full-length clone per slice, reference
transformer_models.py:188), and computes the parameter gradients once over all tokens at the end
(dW = dY_all^T X_all equals the sum over slices of dY_i^T X_i).  Pipeline send/recv, process groups
and the optimizer are not part of this path.
"""
import numpy as np
import torch
import torch.nn as nn

from . import _layer_core as core
from . import _lib
from . import ops
from ._lib import TP_EPI_ACCUMULATE, TP_EPI_STORE, TP_GEMM_TN
from .transformer_models import ModelParallelTransformerLayer, grid_slice_batch_and_sequence


def loss_func(y):
    """Reference terapipe.py:48-49."""
    return torch.mean(y)


def uniform_slice(length, n_slices):
    """Reference utils.py:110-111."""
    return [length // n_slices + int(i < length % n_slices) for i in range(n_slices)]


class TransformerLayers(nn.Module):
    """Reference terapipe.py:52-95.  mixed_precision selects fp16 as the reference does
    (``layer.half()``, terapipe.py:67); ``dtype`` overrides it (bf16 for the 175B/44B shapes).
    accumulate_grads_in_place, defer_weight_grads: see TransformerLayer (layer-level surface only; the fused
    runner takes its parameter gradients once per step either way)."""

    def __init__(self, n_layers, embedding_dim, ffn_embedding_dim, num_attention_heads, mixed_precision=True,
                 dtype=None, device="cuda", activation="relu", accumulate_grads_in_place=False,
                 defer_weight_grads=False):
        super().__init__()
        self.n_layers = n_layers
        self.embedding_dim = embedding_dim
        self.ffn_embedding_dim = ffn_embedding_dim
        self.num_attention_heads = num_attention_heads
        self.mixed_precision = mixed_precision
        self.dtype = dtype if dtype is not None else (torch.float16 if mixed_precision else torch.float32)
        self.device = device
        layers = []
        for _ in range(n_layers):
            layer = ModelParallelTransformerLayer(embedding_dim, ffn_embedding_dim, num_attention_heads,
                                                  device=device, activation=activation)
            layer.accumulate_grads_in_place = accumulate_grads_in_place
            layer.defer_weight_grads = defer_weight_grads
            layers.append(layer.to(self.dtype))
        self.layers = nn.ModuleList(layers)

    def create_cache(self, batch_size, seq_len):
        cache = []
        for layer in self.layers:
            k, v = layer.attn.create_attn_cache(batch_size, seq_len, device=self.device, dtype=self.dtype)
            cache += [k, v]
        return cache

    def forward(self, x, cache, cache_len):
        cache_outputs = []
        for layer_id in range(self.n_layers):
            k_input, v_input = cache[2 * layer_id], cache[2 * layer_id + 1]
            x, (k_output, v_output) = self.layers[layer_id](x, (k_input, v_input), cache_len)
            cache_outputs += [k_output, v_output]
        return x, cache_outputs

    def create_inputs(self, batch_size, seq_len, device="cuda", random=False):
        fn = torch.randn if random else torch.empty
        return fn((seq_len, batch_size, self.embedding_dim), device=device, dtype=self.dtype)


class _StackBuffers:
    """Per-runner device buffers, allocated once and reused by every step: for each batch slice and
    layer the saved activations and the intermediate gradients of the WHOLE sequence, so that a slice
    works on a row range of them (slice i of a [L, Bs, E] tensor is rows [P*Bs, (P+T)*Bs)), the K/V
    caches, the fp32 (or cache-dtype) gradient caches, and the parameter-gradient accumulators."""

    def __init__(self, runner, dtype, device, ws):
        layers = runner.layers
        nl, E, F, H = layers.n_layers, layers.embedding_dim, layers.ffn_embedding_dim, layers.num_attention_heads
        L, Dh = runner.seq_len, layers.embedding_dim // layers.num_attention_heads
        self.dtype, self.device = dtype, device
        # the one-pass dK/dV kernel is 16-bit and has head dimensions 64 and 128; other runs keep gradient caches
        self.position_indexed = runner.suffix_dkdv and dtype != torch.float32 and Dh in (64, 128)
        self.fused_attn_bwd = runner.fused_attn_bwd
        gdt = torch.float32 if runner.fp32_grad_cache else dtype
        kw = dict(dtype=dtype, device=device)
        f32 = dict(dtype=torch.float32, device=device)
        self.per_batch = []
        for Bs in runner.batch_slices:
            R = L * Bs
            b = {}
            b["x"] = [torch.empty(R, E, **kw) for _ in range(nl + 1)]      # x[l] input of layer l; x[nl] output
            b["dx"] = [torch.empty(R, E, **kw) for _ in range(nl + 1)]     # gradient of the same
            for name, width in (("xn", E), ("o", E), ("h", E), ("hn", E), ("a", F),
                                ("dz1", F), ("dhn", E), ("dh", E), ("dqkv", 3 * E), ("dxn", E)):
                b[name] = [torch.empty(R, width, **kw) for _ in range(nl)]
            b["z"] = [torch.empty(R, F, **kw) if layers.layers[l].activation == "gelu" else None for l in range(nl)]
            for name in ("mean1", "rstd1", "mean2", "rstd2"):
                b[name] = [torch.empty(R, **f32) for _ in range(nl)]
            if self.position_indexed:
                # q, lse, delta and dO of every slice, indexed by position like the K/V caches: the dK/dV of
                # a slice's keys are then one pass over all later positions and no gradient cache exists
                b["q"] = [torch.zeros(Bs * H, L, Dh, **kw) for _ in range(nl)]
                b["lse"] = [torch.zeros(Bs * H, L, **f32) for _ in range(nl)]
                b["delta"] = [torch.zeros(Bs * H, L, **f32) for _ in range(nl)]
                b["d_o"] = [torch.zeros(R, E, **kw) for _ in range(nl)]
            else:
                b["q"] = [torch.empty(R, E, **kw) for _ in range(nl)]
                b["lse"] = [torch.empty(R * H, **f32) for _ in range(nl)]
                b["d_o"] = torch.empty(max(runner.seq_slices) * Bs, E, **kw)
                b["delta"] = torch.empty(max(runner.seq_slices) * Bs * H, **f32)
            # zero-filled once: rows beyond the current slice are read only under the causal mask, but
            # they must hold finite values (reference create_attn_cache zero-fills, transformer_models.py:257-261)
            b["cache"] = [torch.zeros(Bs * H, L, Dh, **kw) for _ in range(2 * nl)]
            b["gcache"] = (None if self.position_indexed else
                           [torch.empty(Bs * H, L, Dh, dtype=gdt, device=device) for _ in range(2 * nl)])
            self.per_batch.append(b)
        # parameter-gradient results.  Vector parameters: views of one flat tensor, copied out to autograd
        # with one clone per backward.  Weights: views of one flat tensor that is allocated anew for every
        # backward and handed to autograd as it is (under HIP-graph replay: static, and cloned).
        self.sgrad_layout, n_small = _flat_layout([[(n, ws[l][n].shape) for n in core.SMALL_PARAMS] for l in range(nl)])
        self.wgrad_layout, self.n_big = _flat_layout([[(n, ws[l][n].shape) for n in core.BIG_PARAMS] for l in range(nl)])
        self.sgrad_flat = torch.empty(n_small, **kw)
        self.sgrads = _flat_views(self.sgrad_flat, self.sgrad_layout)
        # their fp32 accumulators in the same layout, so that one launch casts all of them out
        self.small = torch.zeros(n_small, **f32)
        self.small_views = _flat_views(self.small, self.sgrad_layout)
        self.wgrad_flat = None
        self.wgrads = None
        self.wgrad_descs = {}       # (layer, name) -> descriptors of the recorded weight-gradient GEMMs
        self.recording = False
        self.generation = 0         # forward passes run on these buffers
        self.param_ptrs = [t.data_ptr() for w in ws for t in w.values()]
        self.fwd_graph = self.bwd_graph = None
        self.capture_stream = None
        self.states = None
        # launch_replay: 0 = nothing run yet, 1 = one eager pass done (workspaces have their final size),
        # then the recorded program (list) of the pass
        self.fwd_program = self.bwd_program = 0
        self.program_stream = None
        # streams for the slice lanes (see TeraPipe's slice_streams); the gradient-cache mode shares per-slice
        # scratch between layers and stays on one stream
        self.slice_streams = runner.slice_streams
        n = runner.slice_streams if self.position_indexed else 1
        # (lane 0 is the stream the runner is called on: the GPU has few hardware queues per process and two
        # lanes on one queue would run in turn)
        # with lanes, the parameter gradients of a layer run on a stream of their own as soon as the first
        # slice's backward has passed that layer
        pool = _side_streams(device, n) if n > 1 else []
        self.lanes = pool[:n - 1]
        self.dw_stream = pool[n - 1] if n > 1 else None


_SIDE_STREAMS = {}


def _side_streams(device, n):
    """n side streams of `device`, the same ones for every runner of the process.  A process has few hardware
    queues (four by default) and streams are dealt onto them in the order they are made: a second runner with
    fresh streams of its own would find two of its lanes sharing a queue and taking turns (measured: a step of
    140 instead of 105 ms).  A runner's step joins every side stream back into the calling stream before it
    returns, so runners that are stepped one after the other can share them."""
    device = torch.device(device)
    index = device.index if device.index is not None else torch.cuda.current_device()
    pool = _SIDE_STREAMS.setdefault((device.type, index), [])
    while len(pool) < n:
        pool.append(torch.cuda.Stream(device=device))
    return pool[:n]


def _flat_layout(per_layer):
    """[[(name, shape), ...] per layer] -> ([{name: (offset, shape)} per layer], total elements); offsets are
    multiples of 128 elements (256-byte alignment for 16-bit tensors)."""
    out, off = [], 0
    for entries in per_layer:
        d = {}
        for name, shape in entries:
            d[name] = (off, tuple(shape))
            off += (int(np.prod(shape)) + 127) // 128 * 128
        out.append(d)
    return out, off


def _flat_views(flat, layout):
    return [{n: flat[o:o + int(np.prod(s))].view(s) for n, (o, s) in d.items()} for d in layout]


def fused_backward_slices(seq_slices, n_lanes, window=None):
    """[(own_end, fused)] per sequence slice: the end of the positions whose delta a fused attention-backward launch
    of the slice takes itself (the slice and the n_lanes - 1 slices after it, whose launches may still be running),
    and whether the slice's attention backward goes out as that one launch.

    A fused slice records its event BEFORE its launch, so the event does not stand for the delta that the launch
    writes; a two-launch slice reads delta of every later position from memory after waiting for the next slice's
    event only.  With several lanes a two-launch slice may therefore have no fused slice after it -- and since the
    windows shrink towards the end of the sequence, that means all slices fused or none: fused when every slice's
    window is at most `window` positions (ops.FUSED_BWD_WINDOW).  On one stream launches complete in issue order
    and every slice decides for itself."""
    window = ops.FUSED_BWD_WINDOW if window is None else window
    n = max(int(n_lanes), 1)
    L = sum(seq_slices)
    ends, P = [], 0
    for i, T in enumerate(seq_slices):
        ends.append(min(L, P + sum(seq_slices[i:i + n])))
        P += T
    starts = [e - w for e, w in zip(np.cumsum(seq_slices).tolist(), seq_slices)]
    spans = [e - s for e, s in zip(ends, starts)]
    if n == 1:
        return [(e, sp <= window) for e, sp in zip(ends, spans)]
    every = max(spans) <= window
    return [(e, every) for e in ends]


def _program():
    rec = ops.CallRecorder.active
    return rec.program if rec is not None else None


def _wait_stream(waiter, other):
    """waiter.wait_stream(other), noted in the launch program being recorded (if any)."""
    waiter.wait_stream(other)
    prog = _program()
    if prog is not None:
        prog.append((waiter.wait_stream, other))


def _wait_event(stream, event):
    stream.wait_event(event)
    prog = _program()
    if prog is not None:
        prog.append((stream.wait_event, event))


def _record_event(event, stream):
    event.record(stream)
    prog = _program()
    if prog is not None:
        prog.append((event.record, stream))


def _run_program(program):
    """Re-issues a recorded step: every entry is (callable, argument) -- a library call bound to its descriptor
    with the stream handle it was recorded on, or a stream wait / event record."""
    for fn, arg in program:
        if fn(arg):
            raise _lib.TeraPipeHipError("replayed launch failed: %s" % (_lib.load().tp_last_error() or b"").decode())


def _forward_body(runner, ws, act, bufs, states):
    """Every (batch slice, sequence slice) through the whole layer stack, slice-major, reading the batch
    slices from bufs x[0] and leaving the outputs in bufs x[n_layers].  Launches kernels only (no
    allocation, no host synchronisation), so it can be recorded into a HIP graph.

    With slice lanes (bufs.lanes) slice i runs on stream i mod n; the only cross-slice dependency of a layer
    (the attention kernel reads the K/V rows of the earlier slices) is enforced by an event at that point, so
    consecutive slices run through the stack side by side, which keeps the chip busier than one chain of
    short kernels can and lets GEMMs that use the same weight share its way through the caches."""
    layers = runner.layers
    nl, H, E = layers.n_layers, layers.num_attention_heads, layers.embedding_dim
    side = bufs.lanes
    main = torch.cuda.current_stream()
    lanes = [main] + side if side else []
    for st in side:
        _wait_stream(st, main)
    for b, Bs in enumerate(runner.batch_slices):
        pb = bufs.per_batch[b]
        cache = pb["cache"]
        P = 0
        prev_done = None
        for i, T in enumerate(runner.seq_slices):
            r0, r1 = P * Bs, (P + T) * Bs
            sts, done = [], []
            st_i = lanes[i % len(lanes)] if lanes else main
            pending = None
            if runner.slice_timing is not None:
                runner.slice_timing["fwd"].append(_timing_event(main))
            with torch.cuda.stream(st_i):
                for l in range(nl):
                    sync = None
                    if lanes:
                        # the attention of (slice i, layer l) reads the K/V rows that the in_proj GEMMs of the
                        # earlier slices write at layer l: after its own in_proj GEMM the slice waits for the
                        # previous slice's event of that layer, then records its own -- so an event stands
                        # for the in_proj GEMMs of every slice up to its own.  Nothing else ties slices
                        # together: consecutive slices run through a layer side by side, and the GEMMs that
                        # stream the same weight at the same time share its way through the caches.
                        def sync(l=l, st_i=st_i, prev=prev_done, done=done):
                            if prev is not None:
                                _wait_event(st_i, prev[l])
                            ev = torch.cuda.Event()
                            _record_event(ev, st_i)
                            done.append(ev)
                    if bufs.position_indexed:
                        qv, lv, rows = pb["q"][l][:, P:], pb["lse"][l][:, P:], runner.seq_len
                    else:
                        qv, lv, rows = (pb["q"][l][r0:r1].view(Bs * H, T, E // H),
                                        pb["lse"][l][r0 * H:r1 * H].view(Bs * H, T), 0)
                    # a k-split fc2 leaves its partial sums to the next layer's first LayerNorm (same stream,
                    # nothing in between); the last layer finishes its own output
                    bf = core.Bufs(xn=pb["xn"][l][r0:r1], mean1=pb["mean1"][l][r0:r1], rstd1=pb["rstd1"][l][r0:r1],
                                   q=qv, o=pb["o"][l][r0:r1].view(T, Bs, E), lse=lv, q_bh_rows=rows,
                                   stat_bh_rows=rows, h=pb["h"][l][r0:r1], x_pending=pending, defer_out=l + 1 < nl,
                                   mean2=pb["mean2"][l][r0:r1], rstd2=pb["rstd2"][l][r0:r1], hn=pb["hn"][l][r0:r1],
                                   a=pb["a"][l][r0:r1], z=None if pb["z"][l] is None else pb["z"][l][r0:r1],
                                   out=pb["x"][l + 1][r0:r1], sync=sync)
                    _, st = core.layer_fwd(ws[l], pb["x"][l][r0:r1].view(T, Bs, E), H, cache[2 * l], cache[2 * l + 1],
                                           P, act[l], need_state=True, buf=bf)
                    sts.append(st)
                    pending = bf.out_pending
            prev_done = done
            states[b, i] = sts
            if runner.slice_timing is not None:
                runner.slice_timing["fwd"].append(_timing_event(main))
            P += T                                                               # terapipe.py:264
    for st in side:
        _wait_stream(main, st)


def _backward_body(runner, ws, act, bufs, states):
    """Reverse-order slices (terapipe.py:182-191 of the reference) reading the output gradient from bufs
    dx[n_layers], then one weight-gradient GEMM per weight and one reduction per vector parameter over
    all tokens, into bufs.wgrads / bufs.sgrads.  Launches kernels only."""
    layers = runner.layers
    nl, H = layers.n_layers, layers.num_attention_heads
    E, F = layers.embedding_dim, layers.ffn_embedding_dim
    nb, ns = len(runner.batch_slices), len(runner.seq_slices)
    L = runner.seq_len
    ops.zero_(bufs.small)
    side = bufs.lanes
    main = torch.cuda.current_stream()
    lanes = [main] + side if side else []
    early_dw = bool(lanes) and bufs.position_indexed
    finished = [[] for _ in range(nl)]
    for st in side:
        _wait_stream(st, main)
    if early_dw:
        _wait_stream(bufs.dw_stream, main)
    fusion = fused_backward_slices(runner.seq_slices, len(lanes))
    for b in reversed(range(nb)):
        Bs = runner.batch_slices[b]
        pb = bufs.per_batch[b]
        gc = pb["gcache"]
        P = L
        later_done = None
        for i in reversed(range(ns)):
            T = runner.seq_slices[i]
            P -= T
            r0, r1 = P * Bs, (P + T) * Bs
            last = i == ns - 1
            own_end, fuse = fusion[i]
            if runner.slice_timing is not None:
                runner.slice_timing["bwd"].append(_timing_event(main))
            if bufs.position_indexed:
                # slice lanes: layer l of slice i waits for layer l of slice i+1 (whose dO and delta the
                # one-pass dK/dV reads, and through it for every later slice)
                st_i = lanes[i % len(lanes)] if lanes else main
                done = [None] * nl
                with torch.cuda.stream(st_i):
                    for l in reversed(range(nl)):
                        sync = None
                        if lanes:
                            # the one-pass dK/dV of (slice i, layer l) reads dO and delta of every later
                            # slice at layer l.  Two launches: after its own dQ kernel (which leaves its
                            # delta; its dO is older) the slice waits for the next slice's event of that
                            # layer, then records its own.  One fused launch: the same wait and record come
                            # BEFORE the launch (the slice's dO is there, its delta is not), and the launch
                            # takes the delta of its own positions and of the next len(lanes) - 1 slices --
                            # whose fused launches may still be running -- itself; slice i + len(lanes) is an
                            # earlier piece of work of this same stream, and the slices after it are earlier
                            # work of the streams whose events this one has waited for
                            def sync(l=l, st_i=st_i, later=later_done, done=done):
                                if later is not None:
                                    _wait_event(st_i, later[l])
                                done[l] = torch.cuda.Event()
                                _record_event(done[l], st_i)
                        bf = core.Bufs(dz1=pb["dz1"][l][r0:r1], dhn=pb["dhn"][l][r0:r1], dh=pb["dh"][l][r0:r1],
                                       d_o=pb["d_o"][l][r0:r1], dqkv=pb["dqkv"][l][r0:r1], dxn=pb["dxn"][l][r0:r1],
                                       dx=pb["dx"][l][r0:r1], delta=pb["delta"][l][:, P:], sync=sync)
                        core.layer_bwd(ws[l], states[b, i][l], pb["dx"][l + 1][r0:r1].view(T, Bs, E), H, None, None,
                                       False, False, False, activation=act[l], buf=bf,
                                       suffix=dict(q_all=pb["q"][l], d_o_all=pb["d_o"][l], lse_all=pb["lse"][l],
                                                   delta_all=pb["delta"][l], q_end=L,
                                                   o_all=pb["o"][l].view(L, Bs, E) if bufs.fused_attn_bwd else None,
                                                   own_end=own_end, fused=bufs.fused_attn_bwd and fuse))
                        if lanes:
                            # end of (slice, layer): what the parameter gradients of the layer wait for
                            fin = torch.cuda.Event()
                            _record_event(fin, st_i)
                            finished[l].append(fin)
                            if early_dw and b == 0 and i == 0:
                                # the first slice is the last to pass layer l: once every slice has, the
                                # parameter gradients of the layer start, beside the lower layers
                                for ev in finished[l]:
                                    _wait_event(bufs.dw_stream, ev)
                                with torch.cuda.stream(bufs.dw_stream):
                                    _param_grads_layer(runner, bufs, l)
                later_done = done
                if runner.slice_timing is not None:
                    runner.slice_timing["bwd"].append(_timing_event(main))
                continue
            for l in reversed(range(nl)):
                bf = core.Bufs(dz1=pb["dz1"][l][r0:r1], dhn=pb["dhn"][l][r0:r1], dh=pb["dh"][l][r0:r1],
                               d_o=pb["d_o"][:T * Bs], dqkv=pb["dqkv"][l][r0:r1], dxn=pb["dxn"][l][r0:r1],
                               dx=pb["dx"][l][r0:r1], delta=pb["delta"][:T * Bs * H].view(Bs * H, T))
                # the gradient caches need no zero fill: the last slice (processed first) writes every
                # prefix row with '=', the earlier ones add to rows that were written before
                core.layer_bwd(ws[l], states[b, i][l], pb["dx"][l + 1][r0:r1].view(T, Bs, E), H,
                               gc[2 * l], gc[2 * l + 1], accumulate_prefix=not last,
                               has_incoming=not last, zero_slice_rows=False, activation=act[l], buf=bf)
            if runner.slice_timing is not None:
                runner.slice_timing["bwd"].append(_timing_event(main))
    for st in side:
        _wait_stream(main, st)
    if early_dw:
        _wait_stream(main, bufs.dw_stream)
    if runner.slice_timing is not None:
        runner.slice_timing["param"].append(_timing_event(main))
    # parameter gradients over all tokens: dW = dY_all^T X_all (one GEMM per weight and batch slice),
    # bias gradients = column sums of dY_all, LayerNorm gradients from (dy, x, mean, rstd) of all rows
    if not early_dw:
        for l in range(nl):
            _param_grads_layer(runner, bufs, l)
    ops.accum_cast(bufs.sgrad_flat, bufs.small, False)     # every vector-parameter gradient of the stack
    if runner.slice_timing is not None:
        runner.slice_timing["param"].append(_timing_event(main))


def _param_grads_layer(runner, bufs, l):
    layers = runner.layers
    E, F, L = layers.embedding_dim, layers.ffn_embedding_dim, runner.seq_len
    sv = bufs.small_views[l]
    g = bufs.wgrads[l]
    for bi, pb in enumerate(bufs.per_batch):
        R = L * runner.batch_slices[bi]
        epi = TP_EPI_STORE if bi == 0 else TP_EPI_ACCUMULATE
        dy_out = pb["dx"][l + 1]
        # the four weight gradients as one library call: together their tiles fill whole rounds of the CUs
        items, sinks = [], []
        for name, dy, xin, n_out, n_in in (("attn.in_proj.weight", pb["dqkv"][l], pb["xn"][l], 3 * E, E),
                                           ("attn.out_proj.weight", pb["dh"][l], pb["o"][l], E, E),
                                           ("fc1.weight", pb["dz1"][l], pb["hn"][l], F, E),
                                           ("fc2.weight", dy_out, pb["a"][l], E, F)):
            sinks.append(bufs.wgrad_descs.setdefault((l, name), []) if bufs.recording else None)
            items.append((TP_GEMM_TN, dy, xin, n_out, n_in, R, g[name], epi))
        ops.gemm_grouped(items, sinks)
        # the eight vector-parameter gradients of the layer (four bias column sums, two LayerNorm pairs): one launch
        ops.vec_param_grads([(pb["dqkv"][l], sv["attn.in_proj.bias"]),
                             (pb["dh"][l], sv["attn.out_proj.bias"]),
                             (pb["dz1"][l], sv["fc1.bias"]),
                             (dy_out, sv["fc2.bias"]),
                             (pb["dxn"][l], pb["x"][l], pb["mean1"][l], pb["rstd1"][l], sv["attn_ln.weight"], sv["attn_ln.bias"]),
                             (pb["dhn"][l], pb["h"][l], pb["mean2"][l], pb["rstd2"][l], sv["fc_ln.weight"], sv["fc_ln.bias"])])


def _timing_event(stream):
    ev = torch.cuda.Event(enable_timing=True)
    ev.record(stream)
    return ev


def _capture(fn, bufs):
    """Records fn()'s kernel launches into a HIP graph (after the caller has run fn() eagerly once, so
    that every buffer already exists).  The capture runs on a stream the runner keeps for it, and that
    stream's k-split workspace is sized beforehand to what the eager pass needed on the calling stream:
    nothing is allocated while the capture is open."""
    torch.cuda.synchronize()
    dev = torch.device(bufs.device)
    if bufs.capture_stream is None:
        bufs.capture_stream = torch.cuda.Stream(device=dev)
    need = ops.Workspace.size(dev, torch.cuda.current_stream(dev).cuda_stream)
    if need:
        ops.Workspace.get(need, dev, stream=bufs.capture_stream.cuda_stream)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=bufs.capture_stream):
        fn()
    return g


class _TeraPipeFunction(torch.autograd.Function):
    """One autograd node around the whole slice grid (see _forward_body / _backward_body)."""

    @staticmethod
    def forward(ctx, runner, inputs, *flat_params):
        layers = runner.layers
        nl, E = layers.n_layers, layers.embedding_dim
        ws = [dict(zip(core.PARAM_NAMES, flat_params[12 * i:12 * i + 12])) for i in range(nl)]
        act = [l.activation for l in layers.layers]
        bufs = runner._stack_buffers(inputs.dtype, inputs.device, ws)
        nb, ns = len(runner.batch_slices), len(runner.seq_slices)
        b0 = 0
        for b, Bs in enumerate(runner.batch_slices):
            # the batch slice as [L*Bs, E] rows (t, b_local): a copy, as grid_slice_batch_and_sequence makes
            bufs.per_batch[b]["x"][0].view(runner.seq_len, Bs, E).copy_(inputs[:, b0:b0 + Bs, :])
            b0 += Bs
        replayable = runner.launch_replay and ops.CallRecorder.active is None and runner.slice_timing is None
        if runner.use_hip_graph and bufs.fwd_graph is not None:
            bufs.fwd_graph.replay()
            states = bufs.states
        elif replayable and isinstance(bufs.fwd_program, list) and \
                bufs.program_stream == torch.cuda.current_stream().cuda_stream:
            _run_program(bufs.fwd_program)
            states = bufs.states
        elif replayable and bufs.fwd_program == 1:
            # second pass: run it and keep what it launched
            states = np.empty((nb, ns), dtype="O")
            with ops.CallRecorder(program=[]) as rec:
                _forward_body(runner, ws, act, bufs, states)
            bufs.fwd_program, bufs.states = rec.program, states
            bufs.program_stream = torch.cuda.current_stream().cuda_stream
        else:
            if replayable and bufs.fwd_program == 0:
                bufs.fwd_program = 1
            states = np.empty((nb, ns), dtype="O")
            _forward_body(runner, ws, act, bufs, states)
            if runner.use_hip_graph:
                bufs.states = states
                bufs.fwd_graph = _capture(lambda: _forward_body(runner, ws, act, bufs, np.empty((nb, ns), dtype="O")), bufs)
        runner.last_caches = [pb["cache"] for pb in bufs.per_batch]
        if runner.keep_states:
            runner.last_states = states.copy()
        if nb == 1:
            y = bufs.per_batch[0]["x"][nl].view(runner.seq_len, runner.batch_slices[0], E).clone()
        else:
            y = torch.cat([pb["x"][nl].view(runner.seq_len, Bs, E)
                           for pb, Bs in zip(bufs.per_batch, runner.batch_slices)], dim=1)
        # the buffers hold ONE step's activations: a backward must run before the next forward overwrites them
        bufs.generation += 1
        ctx.generation = bufs.generation
        ctx.runner, ctx.ws, ctx.act, ctx.states, ctx.bufs = runner, ws, act, states, bufs
        return y

    @staticmethod
    def backward(ctx, grad_y):
        runner, ws, act, states, bufs = ctx.runner, ctx.ws, ctx.act, ctx.states, ctx.bufs
        if ctx.generation != bufs.generation or bufs is not runner._sbufs:
            raise RuntimeError("TeraPipe keeps the activations of one step in buffers that the next forward "
                               "reuses: this backward belongs to a forward that a later forward has overwritten")
        layers = runner.layers
        nl, E = layers.n_layers, layers.embedding_dim
        L = runner.seq_len
        b0 = 0
        for b, Bs in enumerate(runner.batch_slices):
            bufs.per_batch[b]["dx"][nl].view(L, Bs, E).copy_(grad_y[:, b0:b0 + Bs, :])
            b0 += Bs
        replayable = runner.launch_replay and ops.CallRecorder.active is None and runner.slice_timing is None
        if runner.use_hip_graph:
            if bufs.wgrad_flat is None:      # static storage for the graph
                bufs.wgrad_flat = torch.empty(bufs.n_big, dtype=grad_y.dtype, device=grad_y.device)
                bufs.wgrads = _flat_views(bufs.wgrad_flat, bufs.wgrad_layout)
        else:
            # fresh storage per backward: autograd takes these tensors as the gradients, no copy
            bufs.wgrad_flat = torch.empty(bufs.n_big, dtype=grad_y.dtype, device=grad_y.device)
            bufs.wgrads = _flat_views(bufs.wgrad_flat, bufs.wgrad_layout)
        if runner.use_hip_graph and bufs.bwd_graph is not None:
            bufs.bwd_graph.replay()
        elif replayable and isinstance(bufs.bwd_program, list) and states is bufs.states and \
                bufs.program_stream == torch.cuda.current_stream().cuda_stream:
            for (l, name), descs in bufs.wgrad_descs.items():
                ptr = bufs.wgrads[l][name].data_ptr()
                for d in descs:
                    d.C = ptr
            _run_program(bufs.bwd_program)
        elif replayable and bufs.bwd_program == 1 and states is bufs.states:
            bufs.wgrad_descs, bufs.recording = {}, True
            try:
                with ops.CallRecorder(program=[]) as rec:
                    _backward_body(runner, ws, act, bufs, states)
            finally:
                bufs.recording = False
            bufs.bwd_program = rec.program
        else:
            if replayable and bufs.bwd_program == 0:
                bufs.bwd_program = 1
            _backward_body(runner, ws, act, bufs, states)
            if runner.use_hip_graph:
                bufs.bwd_graph = _capture(lambda: _backward_body(runner, ws, act, bufs, states), bufs)
        # vector-parameter gradients: one clone of the flat buffer (it is reused by the next step); weight
        # gradients: this backward's own storage, or a clone of the graph's static one
        sviews = _flat_views(bufs.sgrad_flat.clone(), bufs.sgrad_layout)
        wviews = _flat_views(bufs.wgrad_flat.clone(), bufs.wgrad_layout) if runner.use_hip_graph else bufs.wgrads
        grads = []
        for l in range(nl):
            for n in core.PARAM_NAMES:
                grads.append(wviews[l][n] if n in wviews[l] else sviews[l][n])
        if not runner.use_hip_graph:
            bufs.wgrad_flat = bufs.wgrads = None
        dinputs = None
        if ctx.needs_input_grad[1]:
            if len(runner.batch_slices) == 1:
                dinputs = bufs.per_batch[0]["dx"][0].view(L, runner.batch_slices[0], E).clone()
            else:
                dinputs = torch.cat([pb["dx"][0].view(L, Bs, E)
                                     for pb, Bs in zip(bufs.per_batch, runner.batch_slices)], dim=1)
        ctx.states = None
        return (None, dinputs) + tuple(grads)


class TeraPipe(nn.Module):
    """Reference terapipe.py:219-271 on a single stage.  ``forward(inputs)`` returns the concatenated
    outputs [seq_len, batch, E]; ``loss(y).backward()`` then runs the reverse-order slice backward and
    leaves the summed-over-slices gradients in the layers' parameters (and in ``inputs.grad`` when the
    input requires grad).

    The per-slice backward leaves the weight and vector-parameter gradients to one reduction over all
    tokens at the end of backward (dW = dY_all^T X_all equals the sum over slices of dY_i^T X_i; the
    layer-level autograd surface in transformer_models.py accumulates per slice instead).
    fp32_grad_cache: keep the cross-slice dK/dV accumulators in fp32 (one rounding when a slice's own
    rows are emitted) instead of the cache dtype the reference uses.
    suffix_dkdv (fp16 / bf16): keep q, lse, delta and dO of every slice in position-indexed buffers and
    compute the dK/dV of a slice's keys, when its backward runs, in one pass over all later query
    positions (every later slice has run its backward by then) -- the same sum that the reference builds
    up through the cache gradients, without gradient caches and their read-modify-write per slice.  With
    False (and always in fp32) the gradient caches are used.
    fused_attn_bwd (with suffix_dkdv): dQ of a slice and the one-pass dK/dV of its keys go out as one launch whose
    two halves run side by side (the first streams the keys before the slice, the second the queries after it)
    instead of two launches one after the other.  The launch recomputes delta of the slice and of the
    slice_streams - 1 slices after it (its window); on one stream a slice is fused when its window is at most
    ops.FUSED_BWD_WINDOW positions, on several streams all slices are fused when every window is, and none otherwise
    (fused_backward_slices says why).  Same results.
    slice_streams (with suffix_dkdv, fp16 / bf16): slice i runs on stream i mod slice_streams.  The attention
    kernel of a layer waits (by event) for the in_proj GEMMs of the earlier slices at that layer, the one-pass
    dK/dV kernel for the dQ kernels of the later slices; nothing else orders slices, so consecutive slices
    run through the stack side by side.  Same kernels, same arguments, same results; the overlap fills the
    chip where one chain of short kernels cannot, and GEMMs that stream the same weight at the same time
    share its way through the caches.  Default 3 (1 under use_hip_graph).
    launch_replay: the first step runs as written, the second also keeps every library call it makes (bound
    descriptor + stream handle) and every stream wait / event record in one list, and later steps re-issue
    that list: the same launches on the same streams without rebuilding descriptors, views and saved state
    (about 11 us of Python per launch otherwise, which bounds a step of short kernels from the host side).
    Works with slice_streams; same conditions as use_hip_graph.
    One step at a time: the buffers hold the activations of the latest forward, so its backward has to run
    before the next forward (a backward of an older forward raises).
    use_hip_graph: after the first (eager) step, record the kernel launches of forward and of backward
    into two HIP graphs and replay them on later steps.  The runner's buffers are static and the
    launches depend only on shapes, so the replays compute the same thing without the per-launch host
    work; parameters must keep their storage (in-place optimizer updates are fine).
    """

    def __init__(self, layers, batch_size, seq_len, batch_slices, seq_slices, batch_dim=1, sequence_dim=0,
                 fp32_grad_cache=True, use_hip_graph=False, suffix_dkdv=True, slice_streams=None, launch_replay=None,
                 fused_attn_bwd=True):
        super().__init__()
        assert sum(batch_slices) == batch_size and sum(seq_slices) == seq_len
        assert batch_dim == 1 and sequence_dim == 0, "layers take [seq, batch, embed] inputs"
        self.batch_size, self.seq_len = batch_size, seq_len
        self.batch_slices, self.seq_slices = list(batch_slices), list(seq_slices)
        self.batch_dim, self.sequence_dim = batch_dim, sequence_dim
        self.layers = layers
        self.fp32_grad_cache = fp32_grad_cache
        self.use_hip_graph = use_hip_graph
        self.suffix_dkdv = suffix_dkdv
        self.fused_attn_bwd = bool(fused_attn_bwd)
        # defaults: three slice streams and launch replay; one stream and no replay under use_hip_graph
        self.slice_streams = int(slice_streams) if slice_streams is not None else (1 if use_hip_graph else 3)
        self.launch_replay = bool(launch_replay) if launch_replay is not None else not use_hip_graph
        self._check_mode()
        # set to {"fwd": [], "bwd": [], "param": []} to have the (eager, single-stream) step bracket every slice's
        # forward and backward and the parameter-gradient tail with timing events (latency_model.py uses it)
        self.slice_timing = None
        self._sbufs = None
        self.last_caches = None
        self.keep_states = False   # debugging / tests: keep the per-slice saved activations of the last forward
        self.last_states = None

    def _check_mode(self):
        """use_hip_graph with slice_streams > 1 is refused: the one run of that combination at full scale
        (24 layers x 8 slices, two lanes) ended in a host segmentation fault between the eager step and the
        first replay, and no cause was found.  launch_replay gives the overlapping runner its low host cost."""
        if self.use_hip_graph and self.slice_streams > 1:
            raise ValueError("TeraPipe: use_hip_graph=True needs slice_streams=1 (HIP-graph capture of the "
                             "multi-stream step is switched off; use launch_replay with slice streams)")

    @property
    def n_batch_slices(self):
        return len(self.batch_slices)

    @property
    def n_input_slices(self):
        return len(self.seq_slices)

    def _stack_buffers(self, dtype, device, ws):
        self._check_mode()          # the attributes can be changed after construction
        ptrs = [t.data_ptr() for w in ws for t in w.values()]
        if (self._sbufs is None or self._sbufs.dtype != dtype or self._sbufs.device != device
                or self._sbufs.slice_streams != self.slice_streams
                or self._sbufs.fused_attn_bwd != self.fused_attn_bwd
                or self._sbufs.param_ptrs != ptrs):     # recorded graphs / launches hold the parameter addresses
            self._sbufs = _StackBuffers(self, dtype, device, ws)
        return self._sbufs

    def forward(self, inputs=None):
        if inputs is None:
            inputs = self.layers.create_inputs(self.batch_size, self.seq_len)
        assert inputs.size(self.sequence_dim) == self.seq_len and inputs.size(self.batch_dim) == self.batch_size
        flat = []
        for layer in self.layers.layers:
            p = layer.param_dict()
            flat += [p[n] for n in core.PARAM_NAMES]
        return _TeraPipeFunction.apply(self, inputs, *flat)
