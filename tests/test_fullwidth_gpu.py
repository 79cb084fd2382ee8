"""Oracle parity at the real width of BASELINE configs 2-5: hidden size, head count, FFN size, dtype and
slice list as the configs state them, on one or two layers of the stack.  The CPU oracle's time is what
bounds the layer count and, for configs 4 and 5, the positions run: config 4 runs the first 1024 of its 2048
positions (8 of its 16 slices of 128 tokens), config 5 the first 512 (16 of its 64 slices of 32 tokens, batch
2) -- every GEMM still has the real extents and the attention kernels the real 96 (batch, head) pairs; the
attention kernels alone are taken to the full prefix lengths at these head counts in test_kernels_gpu.py.

Compared per tensor (max |got - ref| / max |ref| <= 2e-2): the output, the input gradient, the final K/V
caches and all twelve parameter gradients of every layer.  The oracle computes in fp32 from the weights and
inputs already rounded to the kernel dtype, and is given the HIP run's ReLU active set (see the module
docstring of test_layer_gpu.py for why).
"""
import pytest
import torch

import oracle
from tests.util import assert_close, load_params_into

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# name: (layers run, hidden, heads, ffn, positions run, batch, dtype, slices, weight std)
FULL_WIDTH = {
    "C2": (2, 2048, 16, 8192, 2048, 1, torch.float16, [256] * 8, 0.02),
    "C3": (1, 5120, 40, 20480, 2048, 1, torch.float16, [512, 384, 320, 256, 224, 192, 160], 0.02),
    "C4": (1, 12288, 96, 49152, 1024, 1, torch.bfloat16, [128] * 8, 0.006),
    "C5": (1, 6144, 48, 24576, 512, 2, torch.bfloat16, [32] * 16, 0.02),
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


# every config on one stream; the three-stream runner (the default) also against the oracle on C3 and C5 (C2 has its
# own bit-equality test against the single-stream runner, C4 differs from C3 only in extents)
@pytest.mark.parametrize("name,streams", [("C2", 1), ("C3", 1), ("C4", 1), ("C5", 1), ("C3", 3), ("C5", 3)])
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
    yo, dxo, fco = oracle.terapipe_forward_backward(leaf, x.float(), dy.float(), H, [B], ss, relu_masks=masks)
    worst = {}
    worst["y"] = assert_close(y, yo, dtype, name + " y")
    worst["dx"] = assert_close(xd.grad, dxo, dtype, name + " dx")
    for j in range(2 * n_layers):
        worst["cache"] = max(worst.get("cache", 0.0),
                             assert_close(runner.last_caches[0][j], fco[0][j], dtype, name + " final cache %d" % j))
    for l, (layer, p) in enumerate(zip(layers.layers, leaf)):
        for n, t in layer.param_dict().items():
            assert t.grad is not None, "%s layer %d %s has no grad" % (name, l, n)
            worst[n] = max(worst.get(n, 0.0), assert_close(t.grad, p[n].grad, dtype, "%s layer %d d(%s)" % (name, l, n)))
    print("  worst rel err: " + ", ".join("%s %.2e" % kv for kv in worst.items()), flush=True)
