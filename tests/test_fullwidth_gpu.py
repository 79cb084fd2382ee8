"""Oracle parity at the real width of benchmark configs 2-5: hidden size, head count, FFN size, dtype and
slice list as the configs state them, on one or two layers of the stack (the CPU oracle's time bounds the
layer count).  test_full_width_against_the_oracle runs configs 4 and 5 on a prefix of the sequence (the first
1024 of 2048 positions = 8 of 16 slices of 128 tokens; the first 512 = 16 of 64 slices of 32 tokens, batch 2)
with the eager runner on one and on three streams; test_full_length_default_runner_against_the_oracle runs
both at all 2048 positions, and configs 2 and 3 with all their layers (24 and 5: the workloads as the benchmark times
them), through the runner as it is constructed by default (three slice streams, launch replay) and compares the first
step (eager) and the third (re-issued from the recorded launches).

Compared per tensor (max |got - ref| / max |ref| <= 2e-2): the output, the input gradient, the final K/V
caches and all twelve parameter gradients of every layer.  The oracle computes in fp32 from the weights and
inputs already rounded to the kernel dtype, and is given the HIP run's ReLU active set (see the module
docstring of test_layer_gpu.py for why).  That active set is itself checked: wherever the oracle's own fc1
pre-activation is further from zero than 2e-2 of the largest one, the HIP run's unit must be active exactly
when the pre-activation is positive, and at most one unit in a hundred may differ at all.
"""
import pytest
import torch

import oracle
from tests.util import assert_close, load_params_into, reference_style_loop

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# name: (layers run, hidden, heads, ffn, positions run, batch, dtype, slices, weight std)
FULL_WIDTH = {
    "C2": (2, 2048, 16, 8192, 2048, 1, torch.float16, [256] * 8, 0.02),
    "C3": (1, 5120, 40, 20480, 2048, 1, torch.float16, [512, 384, 320, 256, 224, 192, 160], 0.02),
    "C4": (1, 12288, 96, 49152, 1024, 1, torch.bfloat16, [128] * 8, 0.006),
    "C5": (1, 6144, 48, 24576, 512, 2, torch.bfloat16, [32] * 16, 0.02),
    "C4-full": (1, 12288, 96, 49152, 2048, 1, torch.bfloat16, [128] * 16, 0.006),
    "C5-full": (1, 6144, 48, 24576, 2048, 2, torch.bfloat16, [32] * 64, 0.02),
    # configs 3 and 2 as the benchmark times them: every layer
    "C3-full": (5, 5120, 40, 20480, 2048, 1, torch.float16, [512, 384, 320, 256, 224, 192, 160], 0.02),
    "C2-full": (24, 2048, 16, 8192, 2048, 1, torch.float16, [256] * 8, 0.02),
}


def _params(n_layers, E, Fd, dtype, std, seed):
    """Oracle-format fp32 parameters holding dtype-rounded values; biases and LayerNorm parameters are
    randomised too (the benchmark's zeros and ones would hide indexing mistakes)."""
    g = torch.Generator().manual_seed(seed)
    ps = []
    for _ in range(n_layers):
        p = oracle.init_layer_params(E, Fd, std, torch.float32, g)
        for k in p:
            if k.endswith("bias"):
                p[k] = torch.randn(p[k].shape, generator=g) * 0.1
            elif k.endswith("ln.weight"):
                p[k] = 1.0 + 0.2 * torch.randn(p[k].shape, generator=g)
        ps.append({k: v.to(dtype).to(torch.float32) for k, v in p.items()})
    return ps


def _check_active_sets(name, masks, preacts, tol=2e-2):
    """The ReLU active set of the run under test against the sign of the oracle's own pre-activations: equal
    wherever |z| > tol * max |z| (a wrong sign decision in the fused epilogues would differ everywhere), and
    different on at most 1 % of all units (those are the near-zero ones a 16-bit run may round either way)."""
    flipped = total = 0
    for key, per_layer in masks.items():
        for l, (m, z) in enumerate(zip(per_layer, preacts[key])):
            want = z > 0
            diff = m.view_as(want) != want
            clear = z.abs() > tol * z.abs().max()
            bad = int((diff & clear).sum())
            assert bad == 0, "%s slice %s layer %d: %d units with |z| > %.0e max|z| have the wrong ReLU decision" % (
                name, key, l, bad, tol)
            flipped += int(diff.sum())
            total += diff.numel()
    assert flipped <= 0.01 * total, "%s: %d of %d ReLU decisions differ from the oracle's" % (name, flipped, total)
    return flipped / max(total, 1)


def _compare_step(name, tag, runner, layers, y, xd, yo, dxo, fco, leaf, dtype):
    n_layers = len(leaf)
    worst = {}
    worst["y"] = assert_close(y, yo, dtype, "%s %s y" % (name, tag))
    worst["dx"] = assert_close(xd.grad, dxo, dtype, "%s %s dx" % (name, tag))
    for j in range(2 * n_layers):
        worst["cache"] = max(worst.get("cache", 0.0), assert_close(runner.last_caches[0][j], fco[0][j], dtype,
                                                                   "%s %s final cache %d" % (name, tag, j)))
    for l, (layer, p) in enumerate(zip(layers.layers, leaf)):
        for n, t in layer.param_dict().items():
            assert t.grad is not None, "%s %s layer %d %s has no grad" % (name, tag, l, n)
            worst[n] = max(worst.get(n, 0.0),
                           assert_close(t.grad, p[n].grad, dtype, "%s %s layer %d d(%s)" % (name, tag, l, n)))
    print("  %s worst rel err: " % tag + ", ".join("%s %.2e" % kv for kv in worst.items()), flush=True)


# every config on one stream; the three-stream runner (the default) also against the oracle on C3, C4 and C5: on three
# streams C3 never fuses its attention backward, C5 always does, and C4's windows (384 positions, 256 and 128 at the
# sequence end) are the ones a per-slice decision would mix (C2 has its own bit-equality test against the
# single-stream runner)
@pytest.mark.parametrize("name,streams", [("C2", 1), ("C3", 1), ("C4", 1), ("C5", 1), ("C3", 3), ("C4", 3), ("C5", 3)])
def test_full_width_against_the_oracle(name, streams):
    import terapipe_amd as ta
    n_layers, E, H, Fd, L, B, dtype, ss, std = FULL_WIDTH[name]
    assert sum(ss) == L
    print("full width %s: %d layer(s), E=%d H=%d F=%d L=%d B=%d %s streams=%d" % (name, n_layers, E, H, Fd, L, B, dtype, streams),
          flush=True)
    ps = _params(n_layers, E, Fd, dtype, std, seed=41)
    g = torch.Generator().manual_seed(43)
    x = torch.randn(L, B, E, generator=g).to(dtype)
    dy = torch.randn(L, B, E, generator=g).to(dtype)
    layers = ta.TransformerLayers(n_layers, E, Fd, H, dtype=dtype, device=DEV)
    load_params_into(layers, ps, dtype)
    runner = ta.TeraPipe(layers, B, L, [B], ss, slice_streams=streams, launch_replay=False)
    runner.keep_states = True
    xd = x.to(DEV).requires_grad_(True)
    y = runner(xd)
    (y * dy.to(DEV)).sum().backward()
    torch.cuda.synchronize()
    masks = {}
    for i in range(len(ss)):
        masks[(0, i)] = [(st.a > 0).view(st.T, st.B, -1).cpu() for st in runner.last_states[0, i]]
    leaf = [{k: v.clone().requires_grad_(True) for k, v in p.items()} for p in ps]
    preacts = {}
    yo, dxo, fco = oracle.terapipe_forward_backward(leaf, x.float(), dy.float(), H, [B], ss, relu_masks=masks,
                                                    preacts=preacts)
    frac = _check_active_sets(name, masks, preacts)
    print("  ReLU decisions that differ from the oracle's: %.2e of all units" % frac, flush=True)
    _compare_step(name, "eager", runner, layers, y, xd, yo, dxo, fco, leaf, dtype)


@pytest.mark.parametrize("in_place,defer", [(False, False), (True, True)], ids=["autograd-accumulates", "deferred-in-place"])
def test_full_width_layer_surface_against_the_oracle(in_place, defer):
    """Config 3's width and slice list through the LAYER-LEVEL surface under the reference's own loop (one
    autograd graph per slice, cache-gradient hand-off through gradient caches), two steps so that the second
    finds .grad tensors to add to: with per-slice parameter gradients handed to autograd, and with a sequence's
    weight gradients deferred to the backward of its first slice and added to .grad inside the kernels.  The smooth
    activation keeps 16-bit sign flips of the ReLU out of the bound (this surface does not expose its active set)."""
    import terapipe_amd as ta
    n_layers, E, H, Fd, L, B, dtype, ss, std = FULL_WIDTH["C3"]
    print("layer-level surface at C3's width: in_place=%s defer=%s" % (in_place, defer), flush=True)
    ps = _params(n_layers, E, Fd, dtype, std, seed=59)
    g = torch.Generator().manual_seed(61)
    x = torch.randn(L, B, E, generator=g).to(dtype)
    dy = torch.randn(L, B, E, generator=g).to(dtype)
    layers = ta.TransformerLayers(n_layers, E, Fd, H, dtype=dtype, device=DEV, activation="gelu",
                                  accumulate_grads_in_place=in_place, defer_weight_grads=defer)
    load_params_into(layers, ps, dtype)
    for step in (1, 2):
        y, dx, finals, cg = reference_style_loop(layers, x.to(DEV), dy.to(DEV), [B], ss)
    torch.cuda.synchronize()
    leaf = [{k: v.clone().requires_grad_(True) for k, v in p.items()} for p in ps]
    yo, dxo, fco, cgo = oracle.terapipe_forward_backward(leaf, x.float(), dy.float(), H, [B], ss,
                                                         return_cache_grads=True, activation="gelu")
    assert_close(y, yo, dtype, "y")
    assert_close(dx, dxo, dtype, "dx")
    for j in range(2 * n_layers):
        assert_close(finals[0][j], fco[0][j], dtype, "final cache %d" % j)
        for i in range(1, len(ss)):
            assert_close(cg[0][i][j], cgo[0][i][j], dtype, "cache grad slice %d tensor %d" % (i, j))
    for l, (layer, p) in enumerate(zip(layers.layers, leaf)):
        for n, t in layer.param_dict().items():
            # two identical steps accumulated into .grad
            assert_close(t.grad, 2.0 * p[n].grad, dtype, "layer %d d(%s) over two steps" % (l, n))
    assert all(not layer._grad_options.pending for layer in layers.layers), "a deferred sequence was left open"


@pytest.mark.parametrize("name", ["C4-full", "C5-full", "C3-full", "C2-full"])
def test_full_length_default_runner_against_the_oracle(name):
    """All 2048 positions of configs 4 and 5 (one layer) and of configs 2 and 3 with all their layers (24 and 5) -- the
    workloads as the benchmark times them -- through the runner as constructed by default (three slice streams,
    launch replay): inside the runner this is what reaches the forward's key split (from 1024 keys on), the
    one-pass dK/dV over a tail of up to 2016 positions, and (config 5) the fused attention backward on lanes.
    Step 1 runs eagerly, step 2 records, step 3 is re-issued from the record; steps 1 and 3 are each compared
    with the oracle."""
    import terapipe_amd as ta
    n_layers, E, H, Fd, L, B, dtype, ss, std = FULL_WIDTH[name]
    assert sum(ss) == L
    print("full length %s: %d layer(s), E=%d H=%d F=%d L=%d B=%d %s" % (name, n_layers, E, H, Fd, L, B, dtype), flush=True)
    ps = _params(n_layers, E, Fd, dtype, std, seed=47)
    g = torch.Generator().manual_seed(53)
    x = torch.randn(L, B, E, generator=g).to(dtype)
    dy = torch.randn(L, B, E, generator=g).to(dtype)
    layers = ta.TransformerLayers(n_layers, E, Fd, H, dtype=dtype, device=DEV)
    load_params_into(layers, ps, dtype)
    runner = ta.TeraPipe(layers, B, L, [B], ss)
    assert runner.slice_streams == 3 and runner.launch_replay
    runner.keep_states = True
    steps = {}
    for step in (1, 2, 3):
        for t in layers.parameters():
            t.grad = None
        xd = x.to(DEV).requires_grad_(True)
        y = runner(xd)
        (y * dy.to(DEV)).sum().backward()
        torch.cuda.synchronize()
        if step == 1:
            masks = {(0, i): [(st.a > 0).view(st.T, st.B, -1).cpu() for st in runner.last_states[0, i]]
                     for i in range(len(ss))}
        if step != 2:
            steps[step] = (y.detach().cpu(), xd.grad.cpu(), [c.cpu() for c in runner.last_caches[0]],
                           [{n: t.grad.cpu() for n, t in layer.param_dict().items()} for layer in layers.layers])
    assert isinstance(runner._sbufs.fwd_program, list) and isinstance(runner._sbufs.bwd_program, list), \
        "the third step was not re-issued from recorded launches"
    leaf = [{k: v.clone().requires_grad_(True) for k, v in p.items()} for p in ps]
    preacts = {}
    yo, dxo, fco = oracle.terapipe_forward_backward(leaf, x.float(), dy.float(), H, [B], ss, relu_masks=masks,
                                                    preacts=preacts)
    frac = _check_active_sets(name, masks, preacts)
    print("  ReLU decisions that differ from the oracle's: %.2e of all units" % frac, flush=True)
    for step, tag in ((1, "step 1 (eager)"), (3, "step 3 (replayed)")):
        y, dx, caches, grads = steps[step]
        worst = {"y": assert_close(y, yo, dtype, "%s %s y" % (name, tag)),
                 "dx": assert_close(dx, dxo, dtype, "%s %s dx" % (name, tag))}
        for j in range(2 * n_layers):
            worst["cache"] = max(worst.get("cache", 0.0),
                                 assert_close(caches[j], fco[0][j], dtype, "%s %s final cache %d" % (name, tag, j)))
        for l, p in enumerate(leaf):
            for n in grads[l]:
                worst[n] = max(worst.get(n, 0.0), assert_close(grads[l][n], p[n].grad, dtype,
                                                               "%s %s layer %d d(%s)" % (name, tag, l, n)))
        print("  %s worst rel err: " % tag + ", ".join("%s %.2e" % kv for kv in worst.items()), flush=True)
