"""Pins of the CPU oracle (oracle/terapipe_oracle.py).  The reference holds no golden vectors, KATs or
fixtures for this path (its only checks are the two relative invariants restated below), so every
oracle function is pinned against a library routine, a closed form, brute force on tiny inputs, or
torch.autograd.gradcheck in fp64 -- each chosen so that a dropped term, a wrong index or a transposed
operand fails.  Runs on the CPU in seconds."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import terapipe_oracle as oo


def _rnd(*shape, seed=0, dtype=torch.float64):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=dtype)


def test_layer_norm_matches_library_and_closed_form():
    x, w, b = _rnd(5, 3, 16, seed=1) * 3 + 1, _rnd(16, seed=2), _rnd(16, seed=3)
    y = oracle.layer_norm(x, w, b)
    assert torch.allclose(y, F.layer_norm(x, (16,), w, b, 1e-5), atol=1e-12)
    # closed form on one row, biased variance, eps inside the square root
    r = x[2, 1]
    mu = r.sum() / 16
    var = ((r - mu) ** 2).sum() / 16
    assert torch.allclose(y[2, 1], (r - mu) / math.sqrt(var + 1e-5) * w + b, atol=1e-12)
    # the module the reference builds (nn.LayerNorm(E)) has eps 1e-5 and affine parameters
    m = torch.nn.LayerNorm(16).double()
    assert m.eps == 1e-5 and m.elementwise_affine


def test_linear_col_row_and_weight_layout():
    x, W, b = _rnd(4, 2, 6, seed=4), _rnd(10, 6, seed=5), _rnd(10, seed=6)
    ref = F.linear(x, W, b)                       # W stored [out, in]
    assert torch.allclose(oracle.linear_col(x, W, b), ref, atol=1e-12)
    assert torch.allclose(oracle.linear_row(x, W, b), ref, atol=1e-12)
    # brute force one element: y[t,b,j] = sum_k x[t,b,k] W[j,k] + b[j]
    s = sum(x[3, 1, k] * W[7, k] for k in range(6)) + b[7]
    assert abs(ref[3, 1, 7] - s) < 1e-12


def test_split_qkv_per_head_interleave_bruteforce():
    T, B, H, Dh = 3, 2, 4, 5
    qkv = torch.arange(T * B * 3 * H * Dh, dtype=torch.float64).view(T, B, 3 * H * Dh)
    q, k, v = oracle.split_qkv(qkv, H)
    assert q.shape == (B * H, T, Dh)
    for t in range(T):
        for b in range(B):
            for h in range(H):
                for d in range(Dh):
                    base = h * 3 * Dh        # feature j belongs to head j // (3 Dh); [q | k | v] inside
                    assert q[b * H + h, t, d] == qkv[t, b, base + d]
                    assert k[b * H + h, t, d] == qkv[t, b, base + Dh + d]
                    assert v[b * H + h, t, d] == qkv[t, b, base + 2 * Dh + d]
    # NOT [Q_all | K_all | V_all]: that layout would put q of head 1 at column Dh
    assert q[1, 0, 0] == qkv[0, 0, 3 * Dh]


def test_mask_rule_and_neg_inf_equivalence():
    T, P = 4, 3
    m = oracle.causal_prefix_mask(T, P)
    assert m.shape == (T, P + T)
    for t in range(T):
        for j in range(P + T):
            assert m[t, j] == (oracle.NEG_INF if j > P + t else 0)
    assert oracle.NEG_INF == -65504 == torch.finfo(torch.float16).min
    # additive -65504 and true -inf masking agree exactly in fp32 for N(0,1)-scale scores
    s = _rnd(6, T, P + T, seed=7, dtype=torch.float32) * 3
    a = F.softmax(s + m, dim=-1)
    binf = F.softmax(s.masked_fill(m < 0, float("-inf")), dim=-1)
    assert torch.equal(a, binf)


def test_assign_cache_forward_alias_and_backward_zeroing():
    cache = torch.zeros(2, 6, 3, dtype=torch.float64, requires_grad=True)
    val = _rnd(2, 2, 3, seed=8).requires_grad_(True)
    out = oracle.assign_cache(cache, val, 2, 4)
    assert out.data_ptr() == cache.data_ptr()                # alias of the same storage
    assert torch.equal(cache.detach()[:, 2:4], val.detach())  # written in place
    assert cache._version == 0                               # through .data: no version bump
    g = _rnd(2, 6, 3, seed=9)
    out.backward(g)
    assert torch.equal(val.grad, g[:, 2:4])
    expect = g.clone()
    expect[:, 2:4] = 0
    assert torch.equal(cache.grad, expect)


def _attn_bruteforce(q, k, v, P):
    """Per-row Python loops: row t attends to keys [0, P + t]."""
    BH, T, Dh = q.shape
    out = torch.zeros(BH, T, Dh, dtype=q.dtype)
    for bh in range(BH):
        for t in range(T):
            n = P + t + 1
            sc = [sum(q[bh, t, d] * k[bh, j, d] for d in range(Dh)) for j in range(n)]
            mx = max(sc)
            e = [math.exp(float(s - mx)) for s in sc]
            z = sum(e)
            for d in range(Dh):
                out[bh, t, d] = sum(e[j] / z * v[bh, j, d] for j in range(n))
    return out


def test_attention_core_bruteforce_and_sdpa():
    B, H, T, P, Dh = 2, 2, 3, 4, 4
    q, k, v = _rnd(B * H, T, Dh, seed=10), _rnd(B * H, P + T, Dh, seed=11), _rnd(B * H, P + T, Dh, seed=12)
    o = oracle.attention_core(q, k, v, oracle.causal_prefix_mask(T, P, torch.float64), T, B)
    assert o.shape == (T, B, H * Dh)
    brute = _attn_bruteforce(q, k, v, P)
    # [T, B, E] with heads concatenated in order: element (t, b, h*Dh + d) is row (b*H + h, t, d)
    assert torch.allclose(o, brute.transpose(0, 1).reshape(T, B, H * Dh), atol=1e-12)
    # P = 0 equals the library's causal attention
    o0 = oracle.attention_core(q, k[:, :T], v[:, :T], oracle.causal_prefix_mask(T, 0, torch.float64), T, B)
    sd = F.scaled_dot_product_attention(q, k[:, :T], v[:, :T], is_causal=True, scale=1.0)
    assert torch.allclose(o0, sd.transpose(0, 1).reshape(T, B, H * Dh), atol=1e-12)


def test_attention_with_prefix_is_row_block_of_full_sequence():
    """Slice rows [P, S) of full-sequence causal attention == attention of the slice against the cache:
    the invariant both of the reference's checks rely on."""
    E, H, L, B, P, T = 16, 2, 10, 2, 6, 4
    p = {k: v.double() for k, v in oracle.init_layer_params(E, 4 * E, 0.3, generator=torch.Generator().manual_seed(1)).items()}
    p["attn.in_proj.bias"] = _rnd(3 * E, seed=20)
    x = _rnd(L, B, E, seed=13)
    full, _ = oracle.attention_forward(p, "attn.", x, H, None, 0)
    ck, cv = [torch.zeros(B * H, L, E // H, dtype=torch.float64) for _ in range(2)]
    a0, (ck, cv) = oracle.attention_forward(p, "attn.", x[:P], H, (ck, cv), 0)
    a1, (ck, cv) = oracle.attention_forward(p, "attn.", x[P:P + T], H, (ck, cv), P)
    assert torch.allclose(a0, full[:P], atol=1e-12)
    assert torch.allclose(a1, full[P:P + T], atol=1e-12)
    # q is scaled by Dh^-0.5 (a dropped scale changes the result)
    sd = F.scaled_dot_product_attention(*[t for t in oracle.split_qkv(oracle.linear_col(x, p["attn.in_proj.weight"], p["attn.in_proj.bias"]), H)], is_causal=True)
    ref = oracle.linear_row(sd.transpose(0, 1).reshape(L, B, E), p["attn.out_proj.weight"], p["attn.out_proj.bias"])
    assert torch.allclose(full, ref, atol=1e-10)


def test_attention_gradcheck_fp64():
    B, H, T, P, Dh = 1, 2, 3, 4, 4
    q = _rnd(B * H, T, Dh, seed=14).requires_grad_(True)
    k = _rnd(B * H, P + T, Dh, seed=15).requires_grad_(True)
    v = _rnd(B * H, P + T, Dh, seed=16).requires_grad_(True)
    mask = oracle.causal_prefix_mask(T, P, torch.float64)
    assert torch.autograd.gradcheck(lambda a, b, c: oracle.attention_core(a, b, c, mask, T, B), (q, k, v), atol=1e-6)


def test_layer_forward_composition_and_gradcheck():
    E, H, T, B = 8, 2, 3, 1
    g = torch.Generator().manual_seed(3)
    p = {k: (v.double() + 0.1 * torch.randn(v.shape, generator=g, dtype=torch.float64)).requires_grad_(True)
         for k, v in oracle.init_layer_params(E, 2 * E, 0.5, generator=g).items()}
    x = _rnd(T, B, E, seed=17).requires_grad_(True)
    y, none = oracle.layer_forward(p, x, H, None, 0, activation="gelu")
    assert none is None
    # composition spelled with library routines: pre-LN residual block
    h = F.layer_norm(x, (E,), p["attn_ln.weight"], p["attn_ln.bias"])
    a, _ = oracle.attention_forward(p, "attn.", h, H, None, 0)
    h1 = a + x
    z = F.linear(F.layer_norm(h1, (E,), p["fc_ln.weight"], p["fc_ln.bias"]), p["fc1.weight"], p["fc1.bias"])
    ref = F.linear(F.gelu(z), p["fc2.weight"], p["fc2.bias"]) + h1
    assert torch.allclose(y, ref, atol=1e-12)
    yr, _ = oracle.layer_forward(p, x, H, None, 0)            # the reference's ReLU
    refr = F.linear(F.relu(z), p["fc2.weight"], p["fc2.bias"]) + h1
    assert torch.allclose(yr, refr, atol=1e-12)
    names = list(p)
    fn = lambda xx, *ws: oracle.layer_forward(dict(zip(names, ws)), xx, H, None, 0, activation="gelu")[0]
    assert torch.autograd.gradcheck(fn, (x,) + tuple(p[n] for n in names), atol=1e-5)
    # relu_mask equal to the oracle's own active set changes nothing
    zmask = (z > 0)
    ym, _ = oracle.layer_forward(p, x, H, None, 0, relu_mask=zmask)
    assert torch.allclose(ym, yr, atol=1e-12)


def test_gelu_erf_is_library_gelu():
    x = _rnd(50, seed=18) * 3
    assert torch.allclose(oracle.gelu_erf(x), F.gelu(x), atol=1e-12)


def test_embedding_and_vocab_cross_entropy_match_library_and_loops():
    g = torch.Generator().manual_seed(4)
    V, E = 11, 6
    W = _rnd(V, E, seed=5)
    ids = torch.randint(0, V, (4, 3), generator=g)
    assert torch.equal(oracle.embedding(ids, W), F.embedding(ids, W))
    bad = ids.clone(); bad[1, 2] = V + 3; bad[0, 0] = -1          # outside the vocabulary: zero rows
    e = oracle.embedding(bad, W)
    for t in range(4):
        for b in range(3):
            ref = W[bad[t, b]] if 0 <= bad[t, b] < V else torch.zeros(E, dtype=W.dtype)
            assert torch.equal(e[t, b], ref)
    z, tgt = _rnd(4, 3, V, seed=6) * 3, torch.randint(0, V, (4, 3), generator=g)
    loss = oracle.vocab_cross_entropy(z, tgt)
    assert torch.allclose(loss, F.cross_entropy(z.view(-1, V), tgt.view(-1), reduction="none").view(4, 3), atol=1e-12)
    for t in range(4):
        for b in range(3):
            s = sum(math.exp(z[t, b, v].item()) for v in range(V))
            assert abs(loss[t, b].item() - (math.log(s) - z[t, b, tgt[t, b]].item())) < 1e-10
    # gradient of the summed loss: softmax - onehot (what the reference returns as grad_input, :79-99)
    zr = z.clone().requires_grad_(True)
    oracle.vocab_cross_entropy(zr, tgt).sum().backward()
    assert torch.allclose(zr.grad, torch.softmax(z, -1) - F.one_hot(tgt, V).to(z.dtype), atol=1e-12)


@pytest.mark.parametrize("mode,wd", [("l2", 0.0), ("l2", 0.05), ("adamw", 0.05), ("adamw", 0.0)])
def test_adam_step_matches_library_optimizers(mode, wd):
    """torch.optim.Adam is the L2 form, torch.optim.AdamW the decoupled form apex's adam_w_mode selects; six
    steps in float64 so that bias correction and both moments matter."""
    from oracle import optimizer_oracle as opt
    rng = np.random.default_rng(11)
    p0 = rng.standard_normal(257)
    hyper = dict(lr=3e-3, beta1=0.8, beta2=0.95, eps=1e-6, weight_decay=wd)
    pt = torch.tensor(p0, dtype=torch.float64, requires_grad=True)
    cls = torch.optim.Adam if mode == "l2" else torch.optim.AdamW
    lib = cls([pt], lr=hyper["lr"], betas=(hyper["beta1"], hyper["beta2"]), eps=hyper["eps"], weight_decay=wd)
    p, m, v = p0.copy(), np.zeros_like(p0), np.zeros_like(p0)
    for step in range(1, 7):
        g = rng.standard_normal(257) * (0.1 + step)
        pt.grad = torch.tensor(g, dtype=torch.float64)
        lib.step()
        p, m, v = opt.adam_step(p, g, m, v, step, adam_w_mode=(mode == "adamw"), **hyper)
        np.testing.assert_allclose(p, pt.detach().numpy(), rtol=1e-12, atol=1e-14)
    st = lib.state[pt]
    np.testing.assert_allclose(m, st["exp_avg"].numpy(), rtol=1e-12, atol=0)
    np.testing.assert_allclose(v, st["exp_avg_sq"].numpy(), rtol=1e-12, atol=0)
    # without bias correction the first step is lr * (1-b1) g / (sqrt((1-b2) g^2) + eps): closed form
    g = np.array([2.0, -0.5])
    p1, _, _ = opt.adam_step(np.zeros(2), g, np.zeros(2), np.zeros(2), 1, lr=1.0, beta1=0.9, beta2=0.99, eps=0.0,
                             bias_correction=False)
    np.testing.assert_allclose(p1, -np.sign(g) * 0.1 / math.sqrt(0.01), rtol=1e-12)
    # loss-scale path: gradients 128 x larger with loss_scale 128 give the same update, and the model copy
    # is the rounded master
    ma, m2, v2, model = opt.update_weights(p0, 128.0 * g[0] * np.ones(257), np.zeros(257), np.zeros(257), 1, 128.0,
                                           np.float16, lr=1e-2)
    mb, _, _ = opt.adam_step(p0, g[0] * np.ones(257), np.zeros(257), np.zeros(257), 1, lr=1e-2)
    np.testing.assert_array_equal(ma, mb)
    np.testing.assert_array_equal(model, mb.astype(np.float32).astype(np.float16))


def test_slicers():
    assert oracle.uniform_slice(10, 4) == [3, 3, 2, 2]          # first len % n slices get one more
    assert oracle.uniform_slice(128, 8) == [16] * 8
    x = torch.arange(6 * 4 * 2, dtype=torch.float32).view(6, 4, 2)
    g = oracle.grid_slice_batch_and_sequence(x, [1, 3], [2, 4], requires_grad=True)
    assert g.shape == (2, 2) and g.dtype == object
    assert torch.equal(g[1, 1], x[2:6, 1:4]) and g[1, 1].is_contiguous() and g[1, 1].requires_grad and g[1, 1].is_leaf
    with pytest.raises(AssertionError):
        oracle.grid_slice_batch_and_sequence(x, [4], [2, 3])


@pytest.mark.parametrize("bs,ss", [([2], [4, 4, 4, 4]), ([1, 1], [5, 3, 8]), ([2], [16]), ([2], [1] * 16)])
def test_sliced_equals_unsliced_and_cache_grad_contract(bs, ss):
    """Sum over reverse-ordered slices of every gradient == unsliced autograd gradients
    (NCCLTransformerRunner.verify, test_transformer_terapipe.py:333-352; verify_one_step,
    terapipe.py:368-423), and rows >= P_i of the cache-input gradients are zero."""
    n_layers, E, H, L, B = 2, 16, 2, 16, 2
    ps = [{k: v.double() for k, v in p.items()} for p in oracle.init_stack_params(n_layers, E, 4 * E, 0.3, seed=5)]
    for p in ps:
        p["fc1.bias"] = _rnd(4 * E, seed=30) * 0.1
    x, dy = _rnd(L, B, E, seed=19), _rnd(L, B, E, seed=20)
    leaf = [{k: v.clone().requires_grad_(True) for k, v in p.items()} for p in ps]
    y, dx, fc, cg = oracle.terapipe_forward_backward(leaf, x, dy, H, bs, ss, return_cache_grads=True)
    ref = [{k: v.clone().requires_grad_(True) for k, v in p.items()} for p in ps]
    y1, dx1 = oracle.unsliced_forward_backward(ref, x, dy, H)
    assert torch.allclose(y, y1, atol=1e-10) and torch.allclose(dx, dx1, atol=1e-10)
    for a, b in zip(leaf, ref):
        for k in a:
            assert torch.allclose(a[k].grad, b[k].grad, atol=1e-9), k
    for b in range(len(bs)):
        P = 0
        for i, s in enumerate(ss):
            for t in cg[b][i]:
                if i == 0:
                    assert t is None or not t.abs().any()        # nothing precedes the first slice
                else:
                    assert not t[:, P:].abs().any()
                    assert t[:, :P].abs().any()
            P += s
    # final caches hold K/V of the whole sequence: equal to the unsliced projections
    for l in range(n_layers):
        assert fc[0][2 * l].shape == (bs[0] * H, L, E // H)


def test_golden_fixture_c1_regression():
    """Committed vectors of the tiny config (made by tests/golden/make_golden.py from this oracle):
    guards the oracle against silent drift between rounds; the pins above are what make it correct."""
    import os
    path = os.path.join(os.path.dirname(__file__), "golden", "c1_tiny_fp32.npz")
    z = np.load(path)
    cfg = {k: int(z[k]) for k in ("n_layers", "E", "H", "F", "L", "B", "n_slices", "seed")}
    ps = oracle.init_stack_params(cfg["n_layers"], cfg["E"], cfg["F"], 0.02, torch.float32, seed=cfg["seed"])
    g = torch.Generator().manual_seed(cfg["seed"] + 1)
    x = torch.randn(cfg["L"], cfg["B"], cfg["E"], generator=g)
    dy = torch.randn(cfg["L"], cfg["B"], cfg["E"], generator=g)
    leaf = [{k: v.clone().requires_grad_(True) for k, v in p.items()} for p in ps]
    y, dx, fc = oracle.terapipe_forward_backward(leaf, x, dy, cfg["H"], [cfg["B"]],
                                                 oracle.uniform_slice(cfg["L"], cfg["n_slices"]))
    assert np.allclose(y[::7, :, ::5].numpy(), z["y_sub"], rtol=1e-4, atol=1e-5)
    assert np.allclose(dx[::7, :, ::5].numpy(), z["dx_sub"], rtol=1e-4, atol=1e-5)
    assert np.allclose(leaf[0]["fc1.weight"].grad[::16, ::8].numpy(), z["dfc1_sub"], rtol=1e-4, atol=1e-5)
    assert np.allclose(leaf[3]["attn.in_proj.bias"].grad.numpy(), z["dbqkv3"], rtol=1e-4, atol=1e-5)
    assert np.allclose(fc[0][1][::3, ::9, ::4].numpy(), z["vcache0_sub"], rtol=1e-4, atol=1e-5)
