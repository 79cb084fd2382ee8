"""Slice planning for the sliced layer stack: the dynamic program of the reference's latency_model.py
(`planning` :97-152, `evaluate_split` :155-165, the max-latency sweep of `analysis_model` :168-196) on a
latency grid measured on this GPU with the HIP path instead of loaded from the reference's V100 profiles.

The dynamic program itself is native (tp_plan_slices in libterapipe_hip.so, host code); this module
builds the grid, calls it and mirrors the reference's return values.
"""
import ctypes

import numpy as np
import torch

from . import _lib

STEP_GAP = 8          # latency_model.py:13: slice lengths are multiples of this


def planning(latency_grid, total_batch_size, total_seqlen, pipelinelen, max_latency, step_gap=STEP_GAP):
    """Same contract as the reference's `planning`: returns (final_time, [(batch_size, [slice lengths, last
    slice first]), ...]) or (inf, None) when no plan keeps every slice under max_latency."""
    assert total_seqlen % step_gap == 0
    n = total_seqlen // step_gap
    grid = np.ascontiguousarray(latency_grid, dtype=np.float64)
    assert grid.shape[0] >= total_batch_size + 1 and grid.shape[1] == n + 1 and grid.shape[2] == n + 1, grid.shape
    grid = np.ascontiguousarray(grid[:total_batch_size + 1])
    lib = _lib.load()
    final = ctypes.c_double()
    ng = ctypes.c_int()
    gb = (ctypes.c_int * total_batch_size)()
    gn = (ctypes.c_int * total_batch_size)()
    ss = (ctypes.c_int * (total_batch_size * n))()
    _lib.check(lib.tp_plan_slices(grid.ctypes.data, total_batch_size, n, pipelinelen, float(max_latency),
                                  ctypes.byref(final), ctypes.byref(ng), gb, gn, ss), "tp_plan_slices")
    if ng.value == 0:
        return float("inf"), None
    scheme, pos = [], 0
    for i in range(ng.value):
        scheme.append((gb[i], [ss[pos + j] * step_gap for j in range(gn[i])]))
        pos += gn[i]
    return final.value, scheme


def evaluate_split(latency_grid, split_scheme, pipelinelen, step_gap=STEP_GAP, update_time=0.0, layers_per_node=1):
    """latency_model.py:155-165 on a grid: split_scheme lists (batch_size, [slice lengths in sequence order])."""
    total, largest = 0.0, 0.0
    for batch_size, seq_splits in split_scheme:
        cache_len = 0
        for seq_len in seq_splits:
            t = float(latency_grid[batch_size, seq_len // step_gap, cache_len // step_gap])
            total += t
            cache_len += seq_len
            largest = max(largest, t)
    return total + (pipelinelen - 1) * largest + update_time * layers_per_node


def best_plan(latency_grid, total_batch_size, total_seqlen, pipelinelen, step_gap=STEP_GAP, gap=1e-5):
    """The sweep over the largest allowed slice latency of analysis_model (:176-192): returns
    (best_scheme with slices in sequence order, best_latency)."""
    grid = np.asarray(latency_grid, dtype=np.float64)
    cands = np.sort(np.unique(grid[np.isfinite(grid)]))
    best_latency, best_scheme, last = float("inf"), None, 0.0
    for max_latency in cands:
        if max_latency * pipelinelen > best_latency:
            break
        if max_latency - last < gap:
            continue
        last = max_latency
        latency, scheme = planning(grid, total_batch_size, total_seqlen, pipelinelen, max_latency, step_gap)
        if scheme is not None and latency < best_latency:
            best_latency = latency
            best_scheme = [(b, list(reversed(s))) for b, s in scheme]
    return best_scheme, best_latency


def fit_latency_grid(samples, batch_size, seqlen, layers_per_stage=1, step_gap=STEP_GAP):
    """Builds latency_grid[b][s/step][c/step] the way SingleLayerLatency does (latency_model.py:16-45,
    fit_single_layer_model :52-83) from samples {(b, s, c): seconds per layer}: the no-context latency of
    (b, s) from the c = 0 samples (linear interpolation over s between measured lengths), plus a linear
    model in (b*s, b*c, b*s*c) fitted by least squares to the extra time the context costs."""
    n = seqlen // step_gap
    base = np.full((batch_size + 1, n + 1), np.inf)
    for b in range(1, batch_size + 1):
        pts = sorted((s, t) for (bb, s, c), t in samples.items() if bb == b and c == 0)
        if not pts:
            continue
        xs, ys = np.array([p[0] for p in pts], dtype=np.float64), np.array([p[1] for p in pts])
        grid_s = np.arange(1, n + 1) * step_gap
        base[b, 1:] = np.interp(grid_s, xs, ys)
    X, y = [], []
    for (b, s, c), t in samples.items():
        if c > 0 and np.isfinite(base[b, s // step_gap]):
            X.append([b * s, b * c, b * s * c, 1.0])
            y.append(t - base[b, s // step_gap])
    coef = np.linalg.lstsq(np.array(X), np.array(y), rcond=None)[0] if X else np.zeros(4)
    bb, ss, cc = np.meshgrid(np.arange(batch_size + 1), np.arange(n + 1) * step_gap, np.arange(n + 1) * step_gap,
                             indexing="ij")
    ctx = coef[0] * bb * ss + coef[1] * bb * cc + coef[2] * bb * ss * cc + coef[3]
    ctx = np.where(cc > 0, ctx, 0.0)
    # a fitted latency cannot be negative (noisy samples of a launch-bound size can make the linear term so)
    return np.maximum(base[:, :, None] + ctx, 0.0) * layers_per_stage


def measure_layer_latency(layers, batch_size, seqlen, slice_lens, reps=3):
    """Times the layer stack `layers` (a TransformerLayers) on the current GPU through the HIP path and
    returns {(batch_size, s, c): seconds per layer} for every slice length s in slice_lens and every context
    length c = 0, s, 2s, ... < seqlen: for each s the runner steps over the whole sequence cut into slices of
    s tokens (eager, one stream) with timing events around each slice's forward and each slice's backward;
    the parameter-gradient tail of the step, whose work is proportional to the tokens, is shared out by slice
    length.  The same quantity the reference profiles per (batch, seqlen, attention_cache_len)
    (forward_mean + backward_mean, latency_model.py:64-73)."""
    from .terapipe import TeraPipe
    dev = next(layers.parameters()).device
    dt = next(layers.parameters()).dtype
    E = layers.embedding_dim
    out = {}
    for s in slice_lens:
        n = seqlen // s
        slices = [s] * n + ([seqlen - n * s] if seqlen % s else [])
        runner = TeraPipe(layers, batch_size, seqlen, [batch_size], slices, slice_streams=1, launch_replay=False)
        x = torch.randn(seqlen, batch_size, E, device=dev, dtype=dt)
        r = torch.randn(seqlen, batch_size, E, device=dev, dtype=dt)
        acc = np.zeros((reps, n))
        for i in range(reps + 1):
            for p in layers.parameters():
                p.grad = None
            runner.slice_timing = {"fwd": [], "bwd": [], "param": []}
            (runner(x) * r).sum().backward()
            torch.cuda.synchronize()
            tm = runner.slice_timing
            runner.slice_timing = None
            if i == 0:
                continue          # the first step allocates the runner's buffers
            ns = len(slices)
            fwd = [tm["fwd"][2 * k].elapsed_time(tm["fwd"][2 * k + 1]) for k in range(ns)]
            bwd = [tm["bwd"][2 * k].elapsed_time(tm["bwd"][2 * k + 1]) for k in range(ns)][::-1]   # reverse order
            tail = tm["param"][0].elapsed_time(tm["param"][1])
            for k in range(n):
                acc[i - 1, k] = (fwd[k] + bwd[k] + tail * s / seqlen) * 1e-3
        med = np.median(acc, axis=0)
        for k in range(n):
            out[(batch_size, s, k * s)] = float(med[k]) / layers.n_layers
    return out
