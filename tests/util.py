"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

import oracle

TOL = {torch.float32: 1e-5, torch.float16: 2e-2, torch.bfloat16: 2e-2}


def rel_err(got, ref):
    """max |got - ref| / max |ref| -- the per-tensor relative error the parity gate is stated in."""
    got = got.detach().double().cpu()
    ref = ref.detach().double().cpu()
    denom = ref.abs().max().item()
    if denom == 0.0:
        return (got - ref).abs().max().item()
    return (got - ref).abs().max().item() / denom


def assert_close(got, ref, dtype, name, scale=1.0):
    e = rel_err(got, ref)
    tol = TOL[dtype] * scale
    assert e <= tol, "%s: rel err %.3e > %.1e" % (name, e, tol)
    return e


def make_params(n_layers, E, F, dtype, seed=0, std=0.02, rand_small=True):
    """Oracle-format parameter dicts in fp32 holding values already rounded to `dtype`, so that the
    tolerance measures kernel error only.  rand_small also randomises biases and LayerNorm affine
    parameters (the benchmark configs keep them at 0 / 1, which would hide indexing mistakes)."""
    g = torch.Generator().manual_seed(seed)
    ps = []
    for _ in range(n_layers):
        p = oracle.init_layer_params(E, F, std, torch.float32, g)
        if rand_small:
            for k in p:
                if k.endswith("bias"):
                    p[k] = torch.randn(p[k].shape, generator=g) * 0.1
                elif k.endswith("ln.weight"):
                    p[k] = 1.0 + 0.2 * torch.randn(p[k].shape, generator=g)
        ps.append({k: v.to(dtype).to(torch.float32) for k, v in p.items()})
    return ps


def load_params_into(layers_module, ps, dtype):
    """Copies oracle-format parameters into a terapipe_amd TransformerLayers module."""
    with torch.no_grad():
        for layer, p in zip(layers_module.layers, ps):
            for name, t in layer.param_dict().items():
                t.copy_(p[name].to(dtype))


def oracle_run(ps, x, dy, heads, batch_slices, seq_slices, dtype64=False):
    """Runs the oracle's sliced forward/backward on fresh leaf copies; returns y, dx, caches, grads."""
    dt = torch.float64 if dtype64 else torch.float32
    leaf = [{k: v.to(dt).clone().requires_grad_(True) for k, v in p.items()} for p in ps]
    y, dx, caches = oracle.terapipe_forward_backward(leaf, x.to(dt), dy.to(dt), heads, batch_slices, seq_slices)
    grads = [{k: v.grad for k, v in p.items()} for p in leaf]
    return y, dx, caches, grads


def reference_style_loop(layers, x, dy, batch_slices, seq_slices):
    """The slice loop of the reference's TeraPipe.forward + TeraPipeBackwardPassHook.backward
    (terapipe.py:249-264, :182-191) driven through the layer-level autograd surface."""
    import terapipe_amd as ta
    xs = ta.grid_slice_batch_and_sequence(x, batch_slices, seq_slices, requires_grad=True)
    dys = ta.grid_slice_batch_and_sequence(dy, batch_slices, seq_slices)
    nb, ns = len(batch_slices), len(seq_slices)
    cache_inputs = np.empty((nb, ns), dtype="O")
    cache_outputs = np.empty((nb, ns), dtype="O")
    outputs = np.empty((nb, ns), dtype="O")
    finals = []
    for b in range(nb):
        cache = layers.create_cache(batch_slices[b], x.size(0))
        cache_len = 0
        for i in range(ns):
            cache = [c.detach().requires_grad_() for c in cache]
            y, cache_out = layers(xs[b, i], cache, cache_len)
            cache_inputs[b, i], cache_outputs[b, i], outputs[b, i] = cache, cache_out, y
            cache = cache_out
            cache_len += seq_slices[i]
        finals.append([c.detach() for c in cache])
    for b in reversed(range(nb)):
        da = []
        for i in reversed(range(ns)):
            a = list(cache_outputs[b, i]) if i < ns - 1 else []
            torch.autograd.backward([outputs[b, i]] + a, [dys[b, i]] + da)
            da = [t.grad for t in cache_inputs[b, i]]
    y = torch.cat([torch.cat(list(outputs[b]), 0) for b in range(nb)], 1).detach()
    dx = torch.cat([torch.cat([xs[b, i].grad for i in range(ns)], 0) for b in range(nb)], 1)
    cg = [[[t.grad for t in cache_inputs[b, i]] for i in range(ns)] for b in range(nb)]
    return y, dx, finals, cg
