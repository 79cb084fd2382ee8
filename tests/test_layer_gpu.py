"""Layer / stack / sliced-runner parity on the GPU against the CPU oracle (same seeded inputs).

Tolerance (per tensor, max |got - ref| / max |ref|): 1e-5 fp32, 2e-2 fp16/bf16.  For 16-bit runs the
oracle consumes the weights and inputs already rounded to the kernel dtype and computes in fp32.

ReLU in 16 bit: the derivative of relu_ (reference transformer_models.py:282) is discontinuous, and a
16-bit run decides the sign of near-zero pre-activations by its own rounding.  A few in a thousand
elements flip, and each flip moves a gradient entry by its full magnitude: plain PyTorch fp16/bf16 (the
reference's own numerics) is 2e-2 ... 1e-1 away from the fp32 oracle on the gradients behind the ReLU
for exactly this reason (measured; test_relu_flip_error_is_not_worse_than_plain_torch_16bit keeps that
comparison alive).  The 16-bit gradient checks therefore give the oracle the HIP run's ReLU active set
(oracle.layer_forward(relu_mask=...)), which makes the 2e-2 bound measure arithmetic error only; the
fp32 runs (1e-5) and the GeLU runs (2e-2) need no such alignment and cover the same kernels.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from tests.util import TOL, assert_close, load_params_into, make_params, oracle_run, reference_style_loop, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.float16, torch.bfloat16]


def _mods():
    import terapipe_amd
    return terapipe_amd


def _build_layers(ta, n_layers, E, Fd, H, dtype, ps, activation="relu"):
    layers = ta.TransformerLayers(n_layers, E, Fd, H, mixed_precision=(dtype != torch.float32), dtype=dtype,
                                  device=DEV, activation=activation)
    load_params_into(layers, ps, dtype)
    return layers


def _relu_masks_from_states(states):
    """{(b, i): [mask per layer]} with mask = (saved fc1 activation > 0) reshaped [T, B, F], on the CPU."""
    out = {}
    for b in range(states.shape[0]):
        for i in range(states.shape[1]):
            out[(b, i)] = [(st.a > 0).view(st.T, st.B, -1).cpu() for st in states[b, i]]
    return out


def _param_grads(layers):
    return [{n: t.grad for n, t in layer.param_dict().items()} for layer in layers.layers]


def _check_param_grads(got, ref, dtype, tag):
    worst = 0.0
    for l, (g, r) in enumerate(zip(got, ref)):
        for n in r:
            assert g[n] is not None, "%s layer %d %s has no grad" % (tag, l, n)
            worst = max(worst, assert_close(g[n], r[n], dtype, "%s layer %d d(%s)" % (tag, l, n)))
    return worst


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("activation", ["relu", "gelu"])
def test_single_layer_with_prefix(dtype, activation):
    """One layer, one slice, a pre-filled prefix: outputs, the cache rows it writes, and every gradient
    including the cache-input gradients and their zeroed slice rows (transformer_models.py:186-190)."""
    ta = _mods()
    T, B, H, Dh, P, L = 16, 2, 4, 64, 24, 64
    E, Fd = H * Dh, 4 * H * Dh
    ps = make_params(1, E, Fd, dtype, seed=3)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(T, B, E, generator=g).to(dtype)
    kc0, vc0 = torch.randn(B * H, L, Dh, generator=g).to(dtype), torch.randn(B * H, L, Dh, generator=g).to(dtype)
    dy = torch.randn(T, B, E, generator=g).to(dtype)
    dkc, dvc = torch.randn(B * H, L, Dh, generator=g).to(dtype), torch.randn(B * H, L, Dh, generator=g).to(dtype)

    layers = _build_layers(ta, 1, E, Fd, H, dtype, ps, activation)
    layer = layers.layers[0]
    xd = x.to(DEV).requires_grad_(True)
    kd, vd = kc0.to(DEV).clone().requires_grad_(True), vc0.to(DEV).clone().requires_grad_(True)
    y, (k_out, v_out) = layer(xd, (kd, vd), P)
    mask = None
    if dtype != torch.float32 and activation == "relu":
        mask = (y.grad_fn.st.a > 0).view(T, B, Fd).cpu()

    # oracle in fp32
    p32 = {k: v.clone().requires_grad_(True) for k, v in ps[0].items()}
    xo = x.float().clone().requires_grad_(True)
    ko, vo = kc0.float().clone().requires_grad_(True), vc0.float().clone().requires_grad_(True)
    yo, (ko_out, vo_out) = oracle.layer_forward(p32, xo, H, (ko, vo), P, activation=activation, relu_mask=mask)
    torch.autograd.backward([yo, ko_out, vo_out], [dy.float(), dkc.float(), dvc.float()])
    assert k_out.data_ptr() == kd.data_ptr() and v_out.data_ptr() == vd.data_ptr(), "caches are updated in place"
    assert_close(y, yo, dtype, "y")
    assert_close(k_out, ko_out, dtype, "k cache")
    assert_close(v_out, vo_out, dtype, "v cache")
    torch.autograd.backward([y, k_out, v_out], [dy.to(DEV), dkc.to(DEV), dvc.to(DEV)])
    assert_close(xd.grad, xo.grad, dtype, "dx")
    assert_close(kd.grad, ko.grad, dtype, "d k_cache")
    assert_close(vd.grad, vo.grad, dtype, "d v_cache")
    assert (kd.grad[:, P:P + T] == 0).all() and (vd.grad[:, P:P + T] == 0).all()
    _check_param_grads(_param_grads(layers), [{k: v.grad for k, v in p32.items()}], dtype, "single layer")


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_layer_without_cache_is_plain_causal_attention(dtype):
    """full_cache=None path (transformer_models.py:230-234)."""
    ta = _mods()
    T, B, H, Dh = 48, 2, 2, 64
    E, Fd = H * Dh, 2 * H * Dh
    ps = make_params(1, E, Fd, dtype, seed=5)
    g = torch.Generator().manual_seed(2)
    x, dy = torch.randn(T, B, E, generator=g).to(dtype), torch.randn(T, B, E, generator=g).to(dtype)
    layers = _build_layers(ta, 1, E, Fd, H, dtype, ps)
    xd = x.to(DEV).requires_grad_(True)
    y, cache = layers.layers[0](xd)
    assert cache is None
    mask = None if dtype == torch.float32 else (y.grad_fn.st.a > 0).view(T, B, Fd).cpu()
    p32 = {k: v.clone().requires_grad_(True) for k, v in ps[0].items()}
    xo = x.float().clone().requires_grad_(True)
    yo, none = oracle.layer_forward(p32, xo, H, None, 0, relu_mask=mask)
    assert none is None
    yo.backward(dy.float())
    y.backward(dy.to(DEV))
    assert_close(y, yo, dtype, "y")
    assert_close(xd.grad, xo.grad, dtype, "dx")
    _check_param_grads(_param_grads(layers), [{k: v.grad for k, v in p32.items()}], dtype, "no-cache layer")
    with pytest.raises(AssertionError):
        layers.layers[0](xd, None, 4)      # cache_len must be 0 without a cache


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_attention_module_alone(dtype):
    """MultiheadLMAttentionWithCache.forward(x, full_cache, cache_len) with autograd through the caches."""
    ta = _mods()
    T, B, H, Dh, P, L = 8, 1, 2, 128, 8, 24
    E = H * Dh
    ps = make_params(1, E, 4 * E, dtype, seed=9)
    g = torch.Generator().manual_seed(4)
    x, dy = torch.randn(T, B, E, generator=g).to(dtype), torch.randn(T, B, E, generator=g).to(dtype)
    kc0, vc0 = torch.randn(B * H, L, Dh, generator=g).to(dtype), torch.randn(B * H, L, Dh, generator=g).to(dtype)
    p32 = {k: v.clone().requires_grad_(True) for k, v in ps[0].items()}
    xo = x.float().clone().requires_grad_(True)
    ko, vo = kc0.float().clone().requires_grad_(True), vc0.float().clone().requires_grad_(True)
    yo, (ko_out, vo_out) = oracle.attention_forward(p32, "attn.", xo, H, (ko, vo), P)
    yo.backward(dy.float())
    layers = _build_layers(ta, 1, E, 4 * E, H, dtype, ps)
    attn = layers.layers[0].attn
    xd = x.to(DEV).requires_grad_(True)
    kd, vd = kc0.to(DEV).clone().requires_grad_(True), vc0.to(DEV).clone().requires_grad_(True)
    y, (k_out, v_out) = attn(xd, (kd, vd), P)
    y.backward(dy.to(DEV))
    assert_close(y, yo, dtype, "attn y")
    assert_close(xd.grad, xo.grad, dtype, "attn dx")
    assert_close(kd.grad, ko.grad, dtype, "attn d k_cache")
    assert_close(vd.grad, vo.grad, dtype, "attn d v_cache")
    for n in ("attn.in_proj.weight", "attn.in_proj.bias", "attn.out_proj.weight", "attn.out_proj.bias"):
        assert_close(layers.layers[0].param_dict()[n].grad, p32[n].grad, dtype, n)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_attention_module_without_bias(dtype):
    """MultiheadLMAttentionWithCache(bias=False) (reference transformer_models.py:197, :202-203): no bias
    parameters, no bias keys in the state dict, and the projections compute X W^T alone -- against the oracle
    with zero biases."""
    ta = _mods()
    T, B, H, Dh, P, L = 24, 2, 2, 64, 40, 64
    E = H * Dh
    ps = make_params(1, E, 4 * E, dtype, seed=19)
    for n in ("attn.in_proj.bias", "attn.out_proj.bias"):
        ps[0][n] = torch.zeros_like(ps[0][n])
    g = torch.Generator().manual_seed(14)
    x, dy = torch.randn(T, B, E, generator=g).to(dtype), torch.randn(T, B, E, generator=g).to(dtype)
    kc0, vc0 = torch.randn(B * H, L, Dh, generator=g).to(dtype), torch.randn(B * H, L, Dh, generator=g).to(dtype)
    p32 = {k: v.clone().requires_grad_(True) for k, v in ps[0].items()}
    xo = x.float().clone().requires_grad_(True)
    ko, vo = kc0.float().clone().requires_grad_(True), vc0.float().clone().requires_grad_(True)
    yo, _ = oracle.attention_forward(p32, "attn.", xo, H, (ko, vo), P)
    yo.backward(dy.float())
    attn = ta.MultiheadLMAttentionWithCache(E, H, bias=False, device=DEV).to(dtype)
    assert sorted(attn.state_dict()) == ["in_proj.weight", "out_proj.weight"]
    assert [n for n, _ in attn.named_parameters()] == ["in_proj.weight", "out_proj.weight"]
    with torch.no_grad():
        attn.in_proj.weight.copy_(ps[0]["attn.in_proj.weight"].to(dtype))
        attn.out_proj.weight.copy_(ps[0]["attn.out_proj.weight"].to(dtype))
    xd = x.to(DEV).requires_grad_(True)
    kd, vd = kc0.to(DEV).clone().requires_grad_(True), vc0.to(DEV).clone().requires_grad_(True)
    y, (k_out, v_out) = attn(xd, (kd, vd), P)
    y.backward(dy.to(DEV))
    assert_close(y, yo, dtype, "attn y")
    assert_close(xd.grad, xo.grad, dtype, "attn dx")
    assert_close(kd.grad, ko.grad, dtype, "attn d k_cache")
    assert_close(vd.grad, vo.grad, dtype, "attn d v_cache")
    assert_close(attn.in_proj.weight.grad, p32["attn.in_proj.weight"].grad, dtype, "d in_proj.weight")
    assert_close(attn.out_proj.weight.grad, p32["attn.out_proj.weight"].grad, dtype, "d out_proj.weight")


@pytest.mark.parametrize("in_place,defer", [(False, False), (True, False), (False, True), (True, True)],
                         ids=["autograd-accumulates", "grads-in-place", "deferred", "deferred-in-place"])
@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_reference_style_slice_loop(dtype, in_place, defer):
    """Layer-level autograd contract: detach()/requires_grad_() caches per slice, backward with the
    cache-output gradients of the next slice, cache-input .grad as hand-off.  in_place: the slices after the
    first add their parameter gradients to .grad inside the gradient kernels (accumulate_grads_in_place);
    defer: a sequence's weight gradients are taken once, in the backward of its first slice (defer_weight_grads)."""
    ta = _mods()
    n_layers, E, H, L, B = 2, 256, 4, 64, 2
    Fd = 4 * E
    bs, ss = [1, 1], [16, 24, 8, 16]
    # fp32 runs the reference's ReLU; the 16-bit runs use the smooth activation so that the bound is not
    # dominated by ReLU sign flips (see the module docstring)
    act = "relu" if dtype == torch.float32 else "gelu"
    ps = make_params(n_layers, E, Fd, dtype, seed=1)
    g = torch.Generator().manual_seed(7)
    x, dy = torch.randn(L, B, E, generator=g).to(dtype), torch.randn(L, B, E, generator=g).to(dtype)
    leaf = [{k: v.clone().requires_grad_(True) for k, v in p.items()} for p in ps]
    yo, dxo, fco, cgo = oracle.terapipe_forward_backward(leaf, x.float(), dy.float(), H, bs, ss,
                                                         return_cache_grads=True, activation=act)
    layers = _build_layers(ta, n_layers, E, Fd, H, dtype, ps, act)
    for layer in layers.layers:
        layer.accumulate_grads_in_place, layer.defer_weight_grads = in_place, defer
    y, dx, finals, cg = reference_style_loop(layers, x.to(DEV), dy.to(DEV), bs, ss)
    assert_close(y, yo, dtype, "y")
    assert_close(dx, dxo, dtype, "dx")
    for b in range(len(bs)):
        for j in range(2 * n_layers):
            assert_close(finals[b][j], fco[b][j], dtype, "final cache %d/%d" % (b, j))
            for i in range(1, len(ss)):
                P = sum(ss[:i])
                assert_close(cg[b][i][j], cgo[b][i][j], dtype, "cache grad b%d slice %d tensor %d" % (b, i, j))
                assert (cg[b][i][j][:, P:] == 0).all(), "rows >= P of the cache gradient are zero"
    _check_param_grads(_param_grads(layers), [{k: v.grad for k, v in p.items()} for p in leaf], dtype, "ref loop")


@pytest.mark.parametrize("in_place,defer", [(False, False), (True, False), (False, True), (True, True)],
                         ids=["autograd-accumulates", "grads-in-place", "deferred", "deferred-in-place"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
def test_reference_style_slice_loop_on_64_row_multiples(dtype, in_place, defer):
    """The same loop on slices of 128 / 64 / 192 tokens at hidden 512: a slice's four weight gradients meet
    the conditions of the grouped launch (k a multiple of 64), with the store and the accumulate epilogue."""
    ta = _mods()
    n_layers, E, H, L, B = 2, 512, 4, 384, 1
    Fd = 4 * E
    bs, ss = [1], [128, 64, 192]
    ps = make_params(n_layers, E, Fd, dtype, seed=3)
    g = torch.Generator().manual_seed(11)
    x, dy = torch.randn(L, B, E, generator=g).to(dtype), torch.randn(L, B, E, generator=g).to(dtype)
    leaf = [{k: v.clone().requires_grad_(True) for k, v in p.items()} for p in ps]
    yo, dxo, fco, cgo = oracle.terapipe_forward_backward(leaf, x.float(), dy.float(), H, bs, ss,
                                                         return_cache_grads=True, activation="gelu")
    layers = _build_layers(ta, n_layers, E, Fd, H, dtype, ps, "gelu")
    for layer in layers.layers:
        layer.accumulate_grads_in_place, layer.defer_weight_grads = in_place, defer
    y, dx, finals, cg = reference_style_loop(layers, x.to(DEV), dy.to(DEV), bs, ss)
    assert_close(y, yo, dtype, "y")
    assert_close(dx, dxo, dtype, "dx")
    _check_param_grads(_param_grads(layers), [{k: v.grad for k, v in p.items()} for p in leaf], dtype, "ref loop")


def _run_terapipe(ta, layers, x, dy, B, L, bs, ss, keep_states=False, **kw):
    for p in layers.parameters():
        p.grad = None
    kw.setdefault("slice_streams", 1)
    kw.setdefault("launch_replay", False)
    runner = ta.TeraPipe(layers, B, L, bs, ss, **kw)
    runner.keep_states = keep_states
    xd = x.to(DEV).requires_grad_(True)
    y = runner(xd)
    (y * dy.to(DEV)).sum().backward()
    return runner, y.detach(), xd.grad


@pytest.mark.parametrize("fp32gc", [True, False])
def test_terapipe_c1_tiny_fp32(fp32gc):
    """benchmark config 1 (layer stack part): 4 layers, hidden 256, 4 heads, FFN 1024, seq 128, batch 2,
    fp32, 8 slices of 16, reverse-slice backward, tolerance 1e-5."""
    ta = _mods()
    n_layers, E, H, Fd, L, B = 4, 256, 4, 1024, 128, 2
    ss = oracle.uniform_slice(L, 8)
    ps = make_params(n_layers, E, Fd, torch.float32, seed=0)
    g = torch.Generator().manual_seed(0)
    x, dy = torch.randn(L, B, E, generator=g), torch.randn(L, B, E, generator=g)
    yo, dxo, fco, go = oracle_run(ps, x, dy, H, [B], ss)
    layers = _build_layers(ta, n_layers, E, Fd, H, torch.float32, ps)
    runner, y, dx = _run_terapipe(ta, layers, x, dy, B, L, [B], ss, fp32_grad_cache=fp32gc)
    assert_close(y, yo, torch.float32, "y")
    assert_close(dx, dxo, torch.float32, "dx")
    for j in range(2 * n_layers):
        assert_close(runner.last_caches[0][j], fco[0][j], torch.float32, "final cache %d" % j)
    _check_param_grads(_param_grads(layers), go, torch.float32, "C1")


def test_terapipe_c1_tokens_and_cross_entropy():
    """benchmark config 1 end to end: token ids -> embedding -> sliced stack -> LM head -> mean cross
    entropy on random next-token targets.  The embedding / LM head / loss are harness-owned torch ops on
    both sides; the stack between them is the HIP path vs the oracle."""
    ta = _mods()
    n_layers, E, H, Fd, L, B, V = 4, 256, 4, 1024, 128, 2, 50257
    ss = oracle.uniform_slice(L, 8)
    ps = make_params(n_layers, E, Fd, torch.float32, seed=0, rand_small=False)
    g = torch.Generator().manual_seed(123)
    emb = torch.randn(V, E, generator=g) * 0.02
    ids = torch.randint(0, V, (L, B), generator=g)
    tgt = torch.randint(0, V, (L, B), generator=g)

    def head_loss(y, emb_w):
        return F.cross_entropy((y @ emb_w.t()).view(L * B, V), tgt.to(y.device).view(-1))

    # oracle side
    emb_o = emb.clone().requires_grad_(True)
    x_o = F.embedding(ids, emb_o)
    x_leaf = x_o.detach().clone()
    y_tmp = x_leaf.clone().requires_grad_(True)
    leaf = [{k: v.clone().requires_grad_(True) for k, v in p.items()} for p in ps]
    # forward once without grad to get y, then the loss gradient dy, then the sliced backward
    with torch.no_grad():
        h = x_leaf
        cache = oracle.create_cache(n_layers, B, H, L, E // H)
        outs, cl = [], 0
        for s in ss:
            yi, cache = oracle.stack_forward(leaf, h[cl:cl + s], H, cache, cl)
            outs.append(yi)
            cl += s
        y_full = torch.cat(outs, 0)
    y_req = y_full.clone().requires_grad_(True)
    loss_o = head_loss(y_req, emb_o)
    loss_o.backward()
    yo, dxo, _ = oracle.terapipe_forward_backward(leaf, x_leaf, y_req.grad, H, [B], ss)
    x_o.backward(dxo)

    layers = _build_layers(ta, n_layers, E, Fd, H, torch.float32, ps)
    emb_d = emb.to(DEV).requires_grad_(True)
    runner = ta.TeraPipe(layers, B, L, [B], ss)
    y = runner(F.embedding(ids.to(DEV), emb_d))
    loss = head_loss(y, emb_d)
    loss.backward()
    assert abs(loss.item() - loss_o.item()) <= 1e-5 * abs(loss_o.item())
    assert_close(y, yo, torch.float32, "y")
    assert_close(emb_d.grad, emb_o.grad, torch.float32, "d embedding", 2)
    _check_param_grads(_param_grads(layers), [{k: v.grad for k, v in p.items()} for p in leaf], torch.float32, "C1 CE")


def test_terapipe_c1_end_to_end_native_embedding_and_loss():
    """benchmark config 1 end to end with nothing but the HIP path between the token ids and the loss:
    VocabParallelEmbedding -> sliced stack -> tied LM head -> vocab_parallel_cross_entropy -> mean, against
    the oracle (embedding, stack, cross-entropy restatements) in fp32 at 1e-5."""
    ta = _mods()
    n_layers, E, H, Fd, L, B, V = 4, 256, 4, 1024, 128, 2, 50257
    ss = oracle.uniform_slice(L, 8)
    ps = make_params(n_layers, E, Fd, torch.float32, seed=0, rand_small=False)
    g = torch.Generator().manual_seed(321)
    emb = torch.randn(V, E, generator=g) * 0.02
    ids = torch.randint(0, V, (L, B), generator=g)
    tgt = torch.randint(0, V, (L, B), generator=g)
    # oracle: forward without grad for y, the loss gradient dy, then the sliced backward, then the embedding
    emb_o = emb.clone().requires_grad_(True)
    x_o = oracle.embedding(ids, emb_o)
    x_leaf = x_o.detach().clone()
    leaf = [{k: v.clone().requires_grad_(True) for k, v in p.items()} for p in ps]
    with torch.no_grad():
        cache = oracle.create_cache(n_layers, B, H, L, E // H)
        outs, cl = [], 0
        for sl in ss:
            yi, cache = oracle.stack_forward(leaf, x_leaf[cl:cl + sl], H, cache, cl)
            outs.append(yi)
            cl += sl
        y_full = torch.cat(outs, 0)
    y_req = y_full.clone().requires_grad_(True)
    loss_o = oracle.vocab_cross_entropy(y_req.view(L * B, E) @ emb_o.t(), tgt.view(-1)).mean()
    loss_o.backward()
    yo, dxo, _ = oracle.terapipe_forward_backward(leaf, x_leaf, y_req.grad, H, [B], ss)
    x_o.backward(dxo)

    layers = _build_layers(ta, n_layers, E, Fd, H, torch.float32, ps)
    embd = ta.VocabParallelEmbedding(V, E, device=DEV, dtype=torch.float32)
    with torch.no_grad():
        embd.weight.copy_(emb.to(DEV))
    runner = ta.TeraPipe(layers, B, L, [B], ss)
    y = runner(embd(ids.to(DEV)))
    logits = ta.lm_head_logits(y.reshape(L * B, E), embd.weight)
    loss = ta.vocab_parallel_cross_entropy(logits, tgt.to(DEV).view(-1), vocab_size=V).mean()
    loss.backward()
    assert abs(loss.item() - loss_o.item()) <= 1e-5 * abs(loss_o.item())
    assert_close(y, yo, torch.float32, "y")
    assert_close(embd.weight.grad, emb_o.grad, torch.float32, "d embedding (lookup + tied head)", 2)
    _check_param_grads(_param_grads(layers), [{k: v.grad for k, v in p.items()} for p in leaf], torch.float32, "C1 native")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("case", ["uniform", "nonuniform", "fine", "batch_sliced"])
def test_terapipe_16bit_reduced_shapes(dtype, case):
    """Reduced-size versions of benchmark configs 2-5 (head dim 128, N(0,1) inputs, random-projection
    loss): uniform 256-token slices, the non-uniform DP-style slice list, 32-token slices, and a batch
    of 2 cut into two batch slices."""
    ta = _mods()
    H, Dh = 4, 128
    E, Fd = H * Dh, 4 * H * Dh
    n_layers, L, B, bs = 2, 1024, 1, [1]
    if case == "uniform":
        ss = [256] * 4
    elif case == "nonuniform":
        ss = [256, 192, 160, 128, 112, 96, 80]
    elif case == "fine":
        L, B, bs = 512, 2, [2]
        ss = [32] * 16
    else:
        L, B, bs = 512, 2, [1, 1]
        ss = [128] * 4
    ps = make_params(n_layers, E, Fd, dtype, seed=2, rand_small=True)
    g = torch.Generator().manual_seed(17)
    x, dy = torch.randn(L, B, E, generator=g).to(dtype), torch.randn(L, B, E, generator=g).to(dtype)
    layers = _build_layers(ta, n_layers, E, Fd, H, dtype, ps)
    # the one-pass dK/dV over all later positions (default), then the gradient caches in fp32 and in dtype
    for kw in (dict(), dict(suffix_dkdv=False, fp32_grad_cache=True), dict(suffix_dkdv=False, fp32_grad_cache=False)):
        runner, y, dx = _run_terapipe(ta, layers, x, dy, B, L, bs, ss, keep_states=True, **kw)
        # oracle with the ReLU active set of this run (module docstring)
        leaf = [{k: v.clone().requires_grad_(True) for k, v in p.items()} for p in ps]
        yo, dxo, fco = oracle.terapipe_forward_backward(leaf, x.float(), dy.float(), H, bs, ss,
                                                        relu_masks=_relu_masks_from_states(runner.last_states))
        go = [{k: v.grad for k, v in p.items()} for p in leaf]
        tag = "%s %s" % (case, kw)
        assert_close(y, yo, dtype, tag + " y")
        assert_close(dx, dxo, dtype, tag + " dx")
        for b in range(len(bs)):
            for j in range(2 * n_layers):
                assert_close(runner.last_caches[b][j], fco[b][j], dtype, tag + " final cache")
        _check_param_grads(_param_grads(layers), go, dtype, tag)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("Dh", [16, 32, 80, 96])
def test_terapipe_other_head_dims(dtype, Dh):
    """Head dimensions of the reference's model table other than 64 and 128 (transformer_models.py:33-49: 96 for
    megatron-* and gpt3-7hm, 80 for gpt3-2b, 16 for gpt3-175b-megatron), and 32: the runner keeps gradient caches
    there, whatever suffix_dkdv says, and matches the oracle like the other widths."""
    ta = _mods()
    H = 3
    E, Fd = H * Dh, 4 * H * Dh
    n_layers, L, B, bs, ss = 2, 320, 2, [1, 1], [96, 64, 32, 80, 48]
    ps = make_params(n_layers, E, Fd, dtype, seed=4, rand_small=True)
    g = torch.Generator().manual_seed(23)
    x, dy = torch.randn(L, B, E, generator=g).to(dtype), torch.randn(L, B, E, generator=g).to(dtype)
    layers = _build_layers(ta, n_layers, E, Fd, H, dtype, ps)
    for kw in (dict(), dict(fp32_grad_cache=False)):
        runner, y, dx = _run_terapipe(ta, layers, x, dy, B, L, bs, ss, keep_states=True, **kw)
        masks = None if dtype == torch.float32 else _relu_masks_from_states(runner.last_states)
        leaf = [{k: v.clone().requires_grad_(True) for k, v in p.items()} for p in ps]
        yo, dxo, fco = oracle.terapipe_forward_backward(leaf, x.float(), dy.float(), H, bs, ss, relu_masks=masks)
        go = [{k: v.grad for k, v in p.items()} for p in leaf]
        tag = "Dh=%d %s" % (Dh, kw)
        assert_close(y, yo, dtype, tag + " y")
        assert_close(dx, dxo, dtype, tag + " dx")
        for b in range(len(bs)):
            for j in range(2 * n_layers):
                assert_close(runner.last_caches[b][j], fco[b][j], dtype, tag + " final cache")
        _check_param_grads(_param_grads(layers), go, dtype, tag)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
def test_slicing_invariance_full_width(dtype):
    """Size-independent property at a benchmark width (hidden 2048, 16 heads, seq 2048): gradients with 8
    slices equal gradients with one slice (the invariant of test_transformer_terapipe.py:333-352),
    computed entirely by the HIP path."""
    ta = _mods()
    n_layers, E, H, L, B = 2, 2048, 16, 2048, 1
    Fd = 4 * E
    # smooth activation: the two runs round differently, and ReLU sign flips would dominate the bound
    layers = ta.TransformerLayers(n_layers, E, Fd, H, dtype=dtype, device=DEV, activation="gelu")
    g = torch.Generator().manual_seed(5)
    with torch.no_grad():
        for p in layers.parameters():
            if p.dim() == 2:
                p.copy_((torch.randn(p.shape, generator=g) * 0.02).to(dtype))
    x, dy = torch.randn(L, B, E, generator=g).to(dtype), torch.randn(L, B, E, generator=g).to(dtype)
    _, y8, dx8 = _run_terapipe(ta, layers, x, dy, B, L, [B], [256] * 8)
    g8 = [{n: t.grad.clone() for n, t in layer.param_dict().items()} for layer in layers.layers]
    _, y1, dx1 = _run_terapipe(ta, layers, x, dy, B, L, [B], [L])
    g1 = _param_grads(layers)
    assert_close(y8, y1, dtype, "y")
    assert_close(dx8, dx1, dtype, "dx")
    _check_param_grads(g8, g1, dtype, "sliced vs unsliced")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
def test_relu_flip_error_is_not_worse_than_plain_torch_16bit(dtype):
    """Against the UNALIGNED fp32 oracle (ReLU decided by the oracle's own fp32 pre-activations) the HIP
    path is no further away than the reference's own numerics: the same op sequence run by plain PyTorch
    kernels in the same 16-bit dtype on the same inputs (with a 1.5x + 5e-3 margin)."""
    ta = _mods()
    n_layers, E, H, L, B = 2, 512, 4, 512, 1
    Fd, ss = 4 * E, [128] * 4
    ps = make_params(n_layers, E, Fd, dtype, seed=2)
    g = torch.Generator().manual_seed(17)
    x, dy = torch.randn(L, B, E, generator=g).to(dtype), torch.randn(L, B, E, generator=g).to(dtype)
    yo, dxo, _, go = oracle_run(ps, x, dy, H, [B], ss)
    leaf16 = [{k: v.to(dtype).to(DEV).requires_grad_(True) for k, v in p.items()} for p in ps]
    y16, dx16, _ = oracle.terapipe_forward_backward(leaf16, x.to(DEV), dy.to(DEV), H, [B], ss)
    layers = _build_layers(ta, n_layers, E, Fd, H, dtype, ps)
    _, y, dx = _run_terapipe(ta, layers, x, dy, B, L, [B], ss)
    got = _param_grads(layers)
    assert_close(y, yo, dtype, "y")

    def bound(t16, ref):
        return 1.5 * rel_err(t16, ref) + 5e-3

    assert rel_err(dx, dxo) <= bound(dx16, dxo), "dx"
    for l in range(n_layers):
        for n in go[l]:
            e_hip, b = rel_err(got[l][n], go[l][n]), bound(leaf16[l][n].grad, go[l][n])
            assert e_hip <= b, "layer %d d(%s): hip %.3e, plain torch bound %.3e" % (l, n, e_hip, b)


def test_runner_buffers_are_reused_across_steps():
    """The runner keeps its activation / gradient buffers between steps: a second step on different
    inputs must not see anything of the first (fp32, tolerance 1e-5)."""
    ta = _mods()
    n_layers, E, H, Fd, L, B = 2, 256, 4, 1024, 64, 2
    ss = [16, 32, 16]
    ps = make_params(n_layers, E, Fd, torch.float32, seed=4)
    layers = _build_layers(ta, n_layers, E, Fd, H, torch.float32, ps)
    runner = ta.TeraPipe(layers, B, L, [1, 1], ss)
    for seed in (1, 2):
        g = torch.Generator().manual_seed(seed)
        x, dy = torch.randn(L, B, E, generator=g), torch.randn(L, B, E, generator=g)
        yo, dxo, _, go = oracle_run(ps, x, dy, H, [1, 1], ss)
        for p in layers.parameters():
            p.grad = None
        xd = x.to(DEV).requires_grad_(True)
        y = runner(xd)
        (y * dy.to(DEV)).sum().backward()
        assert_close(y, yo, torch.float32, "step %d y" % seed)
        assert_close(xd.grad, dxo, torch.float32, "step %d dx" % seed)
        _check_param_grads(_param_grads(layers), go, torch.float32, "step %d" % seed)


@pytest.mark.parametrize("dtype,streams", [
    (torch.float32, 1), (torch.bfloat16, 1),
    pytest.param(torch.bfloat16, 3, marks=pytest.mark.skip(
        reason="HIP-graph capture of the multi-stream step is switched off (TeraPipe raises): the one run of it at "
               "24 layers x 8 slices ended in a host segmentation fault and no cause was established"))], ids=str)
def test_hip_graph_replays_match_eager(dtype, streams):
    """use_hip_graph=True: step 1 runs eagerly and records, later steps replay the two graphs.  Several
    replays on different inputs, with eager work and synchronisations of the same process in between,
    each checked against an eager runner on the same layers (bit-identical: same kernels, same order)."""
    ta = _mods()
    n_layers, E, H, Fd, L, B = 2, 256, 2, 1024, 96, 2
    bs, ss = [1, 1], [32, 48, 16]
    ps = make_params(n_layers, E, Fd, dtype, seed=6)
    layers = _build_layers(ta, n_layers, E, Fd, H, dtype, ps, "gelu")
    # (with slice lanes the recorded graphs would also hold the cross-stream dependencies)
    graph_runner = ta.TeraPipe(layers, B, L, bs, ss, use_hip_graph=True, slice_streams=streams)
    eager_runner = ta.TeraPipe(layers, B, L, bs, ss, slice_streams=1, launch_replay=False)

    def step(runner, x, dy):
        for p in layers.parameters():
            p.grad = None
        xd = x.clone().requires_grad_(True)
        y = runner(xd)
        (y * dy).sum().backward()
        return y.detach().clone(), xd.grad.clone(), [p.grad.clone() for p in layers.parameters()]

    for seed in range(5):
        g = torch.Generator().manual_seed(100 + seed)
        x = torch.randn(L, B, E, generator=g).to(dtype).to(DEV)
        dy = torch.randn(L, B, E, generator=g).to(dtype).to(DEV)
        ye, dxe, ge = step(eager_runner, x, dy)
        torch.cuda.synchronize()
        junk = (torch.randn(512, 512, device=DEV) @ torch.randn(512, 512, device=DEV)).sum().item()  # eager work between replays
        assert junk == junk
        yg, dxg, gg = step(graph_runner, x, dy)
        torch.cuda.synchronize()
        assert torch.equal(yg, ye), "replay %d: y" % seed
        assert torch.equal(dxg, dxe), "replay %d: dx" % seed
        for a, b in zip(gg, ge):
            # the vector-parameter gradients are summed with atomics: compare to rounding, not bitwise
            assert_close(a, b, dtype, "replay %d: parameter gradient" % seed, 0.05 if dtype == torch.float32 else 1.0)
    assert graph_runner._sbufs.fwd_graph is not None and graph_runner._sbufs.bwd_graph is not None


@pytest.mark.parametrize("dtype,streams", [(torch.float32, 1), (torch.float16, 1), (torch.float16, 3), (torch.bfloat16, 2),
                                           (torch.bfloat16, None)], ids=str)
def test_launch_replay_matches_eager(dtype, streams):
    """launch_replay=True: step 1 runs as written, step 2 also records every library call and stream
    operation, later steps re-issue the recorded list.  Six steps on different inputs (an in-place parameter
    update in between, as an optimizer makes), each checked against an eager runner on the same layers."""
    ta = _mods()
    n_layers, E, H, Fd, L, B = 2, 256, 2, 1024, 96, 2
    bs, ss = [1, 1], [32, 48, 16]
    ps = make_params(n_layers, E, Fd, dtype, seed=16)
    layers = _build_layers(ta, n_layers, E, Fd, H, dtype, ps, "gelu")
    if streams is None:       # the constructor's defaults: three slice streams, launch replay
        replay_runner = ta.TeraPipe(layers, B, L, bs, ss)
        assert replay_runner.slice_streams == 3 and replay_runner.launch_replay
    else:
        replay_runner = ta.TeraPipe(layers, B, L, bs, ss, launch_replay=True, slice_streams=streams)
    eager_runner = ta.TeraPipe(layers, B, L, bs, ss, slice_streams=1, launch_replay=False)

    def step(runner, x, dy):
        for p in layers.parameters():
            p.grad = None
        xd = x.clone().requires_grad_(True)
        y = runner(xd)
        (y * dy).sum().backward()
        return y.detach().clone(), xd.grad.clone(), [p.grad.clone() for p in layers.parameters()]

    for seed in range(6):
        g = torch.Generator().manual_seed(300 + seed)
        x = torch.randn(L, B, E, generator=g).to(dtype).to(DEV)
        dy = torch.randn(L, B, E, generator=g).to(dtype).to(DEV)
        ye, dxe, ge = step(eager_runner, x, dy)
        yr, dxr, gr = step(replay_runner, x, dy)
        torch.cuda.synchronize()
        assert torch.equal(yr, ye), "step %d: y" % seed
        assert torch.equal(dxr, dxe), "step %d: dx" % seed
        for a, b in zip(gr, ge):
            assert_close(a, b, dtype, "step %d: parameter gradient" % seed, 0.05 if dtype == torch.float32 else 1.0)
        with torch.no_grad():
            for p in layers.parameters():
                p.mul_(0.999)
    sb = replay_runner._sbufs
    assert isinstance(sb.fwd_program, list) and isinstance(sb.bwd_program, list) and len(sb.bwd_program) > len(sb.fwd_program) > 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
def test_slice_streams_match_single_stream(dtype):
    """slice_streams > 1 runs consecutive slices on different streams, one layer apart: same kernels and
    arguments, so outputs and input gradients are bit-identical to the single-stream run (the vector-
    parameter gradients are summed with atomics and compared to rounding)."""
    ta = _mods()
    n_layers, E, H, Fd, L, B = 3, 512, 4, 2048, 512, 2
    ss = [128, 32, 96, 64, 64, 128]
    ps = make_params(n_layers, E, Fd, dtype, seed=9)
    layers = _build_layers(ta, n_layers, E, Fd, H, dtype, ps)
    g = torch.Generator().manual_seed(5)
    x, dy = torch.randn(L, B, E, generator=g).to(dtype), torch.randn(L, B, E, generator=g).to(dtype)
    _, y1, dx1 = _run_terapipe(ta, layers, x, dy, B, L, [B], ss)
    g1 = [p.grad.clone() for p in layers.parameters()]
    for n in (2, 4):
        for rep in range(2):
            _, y2, dx2 = _run_terapipe(ta, layers, x, dy, B, L, [B], ss, slice_streams=n)
            torch.cuda.synchronize()
            assert torch.equal(y2, y1), "y with %d lanes" % n
            assert torch.equal(dx2, dx1), "dx with %d lanes" % n
            for a, b in zip([p.grad for p in layers.parameters()], g1):
                assert_close(a, b, dtype, "parameter gradient with %d lanes" % n, 1.0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
def test_fused_attention_backward_matches_two_launches(dtype):
    """The runner with dQ and the one-pass dK/dV of a slice as one launch (the default) against the same runner with
    the two launches one after the other, on one stream and on three (where the launch sits between the wait for
    the later slice's event and the record of the slice's own): outputs and input gradients bit-identical."""
    ta = _mods()
    n_layers, E, H, Fd, L, B = 3, 512, 4, 2048, 512, 2
    ss = [32, 32, 32, 32, 40, 24, 64, 32, 32, 96, 32, 32, 32]      # windows of three slices on both sides of the limit
    ps = make_params(n_layers, E, Fd, dtype, seed=19)
    layers = _build_layers(ta, n_layers, E, Fd, H, dtype, ps)
    g = torch.Generator().manual_seed(15)
    x, dy = torch.randn(L, B, E, generator=g).to(dtype), torch.randn(L, B, E, generator=g).to(dtype)
    _, y1, dx1 = _run_terapipe(ta, layers, x, dy, B, L, [B], ss, fused_attn_bwd=False)
    g1 = [p.grad.clone() for p in layers.parameters()]
    for n in (1, 3):
        for rep in range(2):
            _, y2, dx2 = _run_terapipe(ta, layers, x, dy, B, L, [B], ss, slice_streams=n, fused_attn_bwd=True)
            torch.cuda.synchronize()
            assert torch.equal(y2, y1), "y, fused backward, %d streams" % n
            assert torch.equal(dx2, dx1), "dx, fused backward, %d streams" % n
            for a, b in zip([p.grad for p in layers.parameters()], g1):
                assert_close(a, b, dtype, "parameter gradient, fused backward, %d streams" % n, 1.0)


def test_latency_measurement_feeds_the_planner():
    """measure_layer_latency -> fit_latency_grid -> best_plan on a small stack: every requested point is
    measured, latencies are positive, and the plan covers the sequence (at this size the times are launch
    bound, so nothing is asserted about their order)."""
    ta = _mods()
    from terapipe_amd import latency_model as lm
    n_layers, E, H, Fd, L = 2, 512, 4, 2048, 256
    ps = make_params(n_layers, E, Fd, torch.float16, seed=1)
    layers = _build_layers(ta, n_layers, E, Fd, H, torch.float16, ps)
    samples = lm.measure_layer_latency(layers, 1, L, [32, 64, 128, 256], reps=2)
    assert set(samples) == ({(1, 32, c) for c in range(0, L, 32)} | {(1, 64, c) for c in range(0, L, 64)} |
                            {(1, 128, 0), (1, 128, 128), (1, 256, 0)})
    assert all(t > 0 and t == t for t in samples.values())
    grid = lm.fit_latency_grid(samples, 1, L, layers_per_stage=n_layers)
    scheme, latency = lm.best_plan(grid, 1, L, pipelinelen=4)
    assert scheme is not None and sum(scheme[0][1]) == L and latency >= 0 and latency == latency


def test_planned_and_uniform_slices_run_as_the_latency_grid_predicts():
    """Plan -> run -> predicted against measured (the reference's evaluate_split, latency_model.py:155-163) on two
    layers of the GPT-3 13B width (hidden 5120, 40 heads, FFN 20480, fp16), 1024 positions: the latency grid is
    measured through the HIP path at slice lengths that are multiples of 64, the planner picks the slices for an
    8-stage pipeline on that grid, and both its plan and the uniform 4 x 256 plan are then run on this stage; the
    sum of the grid's slice latencies (pipeline length 1: what one stage spends on a sequence) is within 10 % of the
    measured step in both cases."""
    ta = _mods()
    from terapipe_amd import latency_model as lm
    dtype = torch.float16
    n_layers, E, H, Fd, L, step = 2, 5120, 40, 20480, 1024, 64
    layers = ta.TransformerLayers(n_layers, E, Fd, H, dtype=dtype, device=DEV)
    g = torch.Generator(device=DEV).manual_seed(3)
    with torch.no_grad():
        for p in layers.parameters():
            if p.dim() == 2:
                p.copy_((torch.randn(p.shape, generator=g, device=DEV) * 0.02).to(dtype))
    lens = [64, 128, 192, 256, 320, 384, 448, 512, 640, 768, 1024]
    samples = lm.measure_layer_latency(layers, 1, L, lens, reps=3)
    assert all(t > 0 and t == t for t in samples.values())
    grid = lm.fit_latency_grid(samples, 1, L, layers_per_stage=n_layers, step_gap=step)
    scheme, planned_latency = lm.best_plan(grid, 1, L, pipelinelen=8, step_gap=step)
    assert scheme is not None and sum(scheme[0][1]) == L and all(s % step == 0 for s in scheme[0][1])
    uniform = [256] * 4
    # the planner's optimum is no worse than the uniform plan on the grid it was given
    assert planned_latency <= lm.evaluate_split(grid, [(1, uniform)], 8, step_gap=step) * (1 + 1e-9)
    x = torch.randn(L, 1, E, generator=g, device=DEV).to(dtype)
    r = torch.randn(L, 1, E, generator=g, device=DEV).to(dtype)
    for name, slices in (("planned", scheme[0][1]), ("uniform", uniform)):
        predicted = lm.evaluate_split(grid, [(1, slices)], 1, step_gap=step)
        runner = ta.TeraPipe(layers, 1, L, [1], slices, slice_streams=1, launch_replay=False)
        times = []
        for i in range(5):
            for p in layers.parameters():
                p.grad = None
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            (runner(x) * r).sum().backward()
            e1.record()
            torch.cuda.synchronize()
            if i:
                times.append(e0.elapsed_time(e1) * 1e-3)
        measured = float(np.median(times))
        print("%s slices %s: predicted %.3f ms, measured %.3f ms" % (name, slices, predicted * 1e3, measured * 1e3), flush=True)
        assert abs(predicted - measured) <= 0.10 * measured, \
            "%s plan %s: predicted %.3f ms, measured %.3f ms" % (name, slices, predicted * 1e3, measured * 1e3)


def test_replay_survives_a_larger_workspace_on_the_same_stream():
    """A recorded step holds its k-split workspaces: a larger k-split GEMM on the same stream between two
    re-issued steps makes the workspace pool grow, and the re-issued step must still write its partial sums into
    memory that is its own (results equal to an eager runner's, step by step)."""
    ta = _mods()
    from terapipe_amd import _lib as L, ops
    dtype = torch.float16
    n_layers, E, H, Fd, Ls, B = 2, 256, 2, 1024, 128, 1
    ss = [32, 64, 32]
    ps = make_params(n_layers, E, Fd, dtype, seed=44)
    layers = _build_layers(ta, n_layers, E, Fd, H, dtype, ps)
    fast = ta.TeraPipe(layers, B, Ls, [B], ss, slice_streams=1, launch_replay=True)
    plain = ta.TeraPipe(layers, B, Ls, [B], ss, slice_streams=1, launch_replay=False)

    def step(runner, seed):
        g = torch.Generator().manual_seed(seed)
        x = torch.randn(Ls, B, E, generator=g).to(dtype).to(DEV)
        dy = (torch.randn(Ls, B, E, generator=g) * 0.1).to(dtype).to(DEV)
        for p in layers.parameters():
            p.grad = None
        xd = x.clone().requires_grad_(True)
        y = runner(xd)
        (y * dy).sum().backward()
        return y.detach().clone(), xd.grad.clone(), [p.grad.clone() for p in layers.parameters()]

    def check(seed, tag):
        y0, dx0, g0 = step(plain, seed)
        y1, dx1, g1 = step(fast, seed)
        torch.cuda.synchronize()
        assert torch.equal(y1, y0), tag + " y"
        assert torch.equal(dx1, dx0), tag + " dx"
        for a, b in zip(g1, g0):
            assert_close(a, b, dtype, tag + " parameter gradient", 1.0)

    for seed in (1, 2, 3):                 # as written, recorded, re-issued
        check(seed, "step %d" % seed)
    assert isinstance(fast._sbufs.fwd_program, list)
    dev = torch.device(DEV)
    stream = torch.cuda.current_stream().cuda_stream
    before = ops.Workspace.size(dev, stream)
    # a k-split product on the same stream that needs more workspace than anything so far
    M, K, ks = 512, 2048, 8
    N = max(4096, (before // (ks * M * 4) // 256 + 1) * 256)     # whatever earlier tests left the pool at
    assert ks * M * N * 4 > before
    A = (torch.randn(M, K, device=DEV) * K ** -0.5).to(dtype)
    Bm = torch.randn(N, K, device=DEV).to(dtype)
    C = torch.empty(M, N, dtype=dtype, device=DEV)
    ops.gemm(L.TP_GEMM_NT, A, Bm, M, N, K, C=C, ksplit=ks)
    assert ops.Workspace.size(dev, stream) >= ks * M * N * 4 > before
    # memory that torch may now hand out: were the old workspace freed, these tensors would land in it
    junk = [torch.full((before // 4 + 1,), float("nan"), device=DEV) for _ in range(4)]
    check(4, "re-issued step after the workspace grew")
    check(5, "second re-issued step after the workspace grew")
    assert all(torch.isnan(j).all() for j in junk), "a re-issued launch wrote into memory it no longer owns"
    assert_close(C, A.float() @ Bm.float().t(), dtype, "the large product itself")


@pytest.mark.parametrize("n_layers,steps", [(2, 5), (24, 4)])
def test_default_runner_matches_single_stream_at_c2_shape(n_layers, steps):
    """benchmark config 2's geometry (hidden 2048, 16 heads, FFN 8192, sequence 2048 as 8 x 256, fp16) on two
    layers and on all 24: the constructor's defaults (three slice streams, launch replay) against one stream
    launched from Python, several steps -- the first as written, the second recorded, the rest re-issued.  Same
    kernels on the same data: outputs and input gradients are bit-identical; the parameter gradients (fp32
    atomics for the vector parameters) agree to rounding."""
    ta = _mods()
    dtype = torch.float16
    E, H, Fd, L, B = 2048, 16, 8192, 2048, 1
    ss = [256] * 8
    print("C2 geometry, %d layers, %d steps" % (n_layers, steps), flush=True)
    if n_layers <= 2:
        ps = make_params(n_layers, E, Fd, dtype, seed=21)
        layers = _build_layers(ta, n_layers, E, Fd, H, dtype, ps)
    else:
        # (the full stack's parameters are drawn on the device: 1.2 G values)
        layers = ta.TransformerLayers(n_layers, E, Fd, H, dtype=dtype, device=DEV)
        gd = torch.Generator(device=DEV).manual_seed(21)
        with torch.no_grad():
            for layer in layers.layers:
                for name, t in layer.param_dict().items():
                    if name.endswith("ln.weight"):
                        t.copy_(1.0 + 0.2 * torch.randn(t.shape, generator=gd, device=DEV))
                    else:
                        t.copy_(torch.randn(t.shape, generator=gd, device=DEV) * (0.1 if name.endswith("bias") else 0.02))
    fast = ta.TeraPipe(layers, B, L, [B], ss)
    plain = ta.TeraPipe(layers, B, L, [B], ss, slice_streams=1, launch_replay=False)
    assert fast.slice_streams == 3 and fast.launch_replay

    def step(runner, x, dy):
        for p in layers.parameters():
            p.grad = None
        xd = x.clone().requires_grad_(True)
        y = runner(xd)
        (y * dy).sum().backward()
        return y.detach().clone(), xd.grad.clone(), [p.grad.clone() for p in layers.parameters()]

    for seed in range(steps):
        g = torch.Generator().manual_seed(700 + seed)
        x = torch.randn(L, B, E, generator=g).to(dtype).to(DEV)
        dy = (torch.randn(L, B, E, generator=g) * 0.1).to(dtype).to(DEV)
        y0, dx0, g0 = step(plain, x, dy)
        y1, dx1, g1 = step(fast, x, dy)
        torch.cuda.synchronize()
        assert torch.equal(y1, y0), "step %d: y" % seed
        assert torch.equal(dx1, dx0), "step %d: dx" % seed
        for a, b in zip(g1, g0):
            assert_close(a, b, dtype, "step %d: parameter gradient" % seed, 1.0)


def test_default_runner_usage_patterns():
    """The constructor's defaults (three slice streams, launch replay) through what a training script does
    besides forward + backward: evaluation passes under no_grad between training steps, a forward that is never
    differentiated, an input that needs no gradient, an optimizer step in place, a parameter whose storage is
    replaced.  Every result against a single-stream runner launched from Python on the same layers."""
    ta = _mods()
    dtype = torch.float16
    n_layers, E, H, Fd, L, B = 2, 256, 2, 1024, 128, 2
    bs, ss = [1, 1], [32, 64, 32]
    ps = make_params(n_layers, E, Fd, dtype, seed=33)
    layers = _build_layers(ta, n_layers, E, Fd, H, dtype, ps)
    fast = ta.TeraPipe(layers, B, L, bs, ss)
    plain = ta.TeraPipe(layers, B, L, bs, ss, slice_streams=1, launch_replay=False)

    def data(seed):
        g = torch.Generator().manual_seed(seed)
        return (torch.randn(L, B, E, generator=g).to(dtype).to(DEV),
                (torch.randn(L, B, E, generator=g) * 0.1).to(dtype).to(DEV))

    def train(runner, x, dy, input_grad=True):
        for p in layers.parameters():
            p.grad = None
        xd = x.clone().requires_grad_(input_grad)
        y = runner(xd)
        (y * dy).sum().backward()
        return y.detach().clone(), (xd.grad.clone() if input_grad else None), [p.grad.clone() for p in layers.parameters()]

    def same_train(seed, input_grad=True, tag=""):
        x, dy = data(seed)
        y0, dx0, g0 = train(plain, x, dy, input_grad)
        y1, dx1, g1 = train(fast, x, dy, input_grad)
        torch.cuda.synchronize()
        assert torch.equal(y1, y0), tag + " y"
        if input_grad:
            assert torch.equal(dx1, dx0), tag + " dx"
        for a, b in zip(g1, g0):
            assert_close(a, b, dtype, tag + " parameter gradient", 1.0)

    def same_eval(seed, tag=""):
        x, _ = data(seed)
        with torch.no_grad():
            y0 = plain(x).clone()
            y1 = fast(x).clone()
        torch.cuda.synchronize()
        assert torch.equal(y1, y0), tag + " y (no_grad)"

    same_eval(1, "eval before any training step")
    same_train(2, tag="step 1")
    same_eval(3, "eval after step 1")
    same_train(4, tag="step 2 (recorded)")
    same_eval(5, "eval after the recording")
    same_train(6, tag="step 3 (re-issued)")
    # a forward that is never differentiated, then a full step
    x, _ = data(7)
    y = fast(x.clone().requires_grad_(True))
    del y
    same_train(8, tag="step after an abandoned forward")
    same_train(9, input_grad=False, tag="input without gradient")
    same_train(10, tag="input with gradient again")
    with torch.no_grad():
        for p in layers.parameters():
            p.add_(torch.randn_like(p) * 1e-3)
    same_train(11, tag="after an in-place update")
    # a parameter that moves to new storage (e.g. a checkpoint load that rebinds .data)
    p0 = next(iter(layers.parameters()))
    p0.data = p0.data.clone()
    same_train(12, tag="after a parameter moved")
    same_train(13, tag="second step after the move")
    same_eval(14, "eval at the end")


def test_backward_of_an_overwritten_forward_raises():
    ta = _mods()
    dtype = torch.float16
    n_layers, E, H, Fd, L, B = 1, 128, 2, 256, 64, 1
    ps = make_params(n_layers, E, Fd, dtype, seed=2)
    layers = _build_layers(ta, n_layers, E, Fd, H, dtype, ps)
    runner = ta.TeraPipe(layers, B, L, [B], [32, 32])
    x = torch.randn(L, B, E).to(dtype).to(DEV).requires_grad_(True)
    y_old = runner(x)
    y_new = runner(x)
    with pytest.raises(RuntimeError, match="overwritten"):
        y_old.sum().backward()
    y_new.sum().backward()            # the latest forward is still intact
    assert x.grad is not None
