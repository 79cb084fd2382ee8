"""Plain-PyTorch CPU restatement (fp32 / fp64) of the reference's sliced GPT-layer path.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Every function cites the reference lines it follows (paths relative to the
reference checkout).  The restatement is functional (weights live in a plain
dict keyed by the reference's state-dict names) and uses ``torch.autograd``
for the backward pass exactly where the reference does.

How each function is pinned (see tests/test_oracle_pins.py):
  layer_norm            -- torch.nn.functional.layer_norm (library routine) and the closed form
  linear_col/linear_row -- fp64 matmul + bias
  split_qkv             -- explicit per-element Python loops over (t, b, h, d)
  causal_prefix_mask    -- brute-force per-element rule; -65504 vs -inf equivalence in fp32
  attention_core        -- F.scaled_dot_product_attention(is_causal=True) for P = 0; row block
                           [P, S) of the full-sequence causal result for P > 0; per-row Python
                           softmax loops on tiny shapes; torch.autograd.gradcheck in fp64
  assign_cache          -- brute-force check of forward aliasing + backward zeroing rule
  layer_forward         -- composition of the above; sliced == unsliced invariant that the
                           reference's own checks rely on (test_transformer_terapipe.py:333-352)
  terapipe_forward_backward -- sum over reverse-ordered slices == unsliced autograd gradients
                           (same invariant, terapipe.py:368-423); grad-cache rows >= P are zero
Absolute pin: torch 2.10 CPU kernels in fp64.  The reference holds no golden vectors for this
path, so in absolute terms its own numbers are "parity unpinned"; the relative invariants above
are the ones its checks use.
"""
import math
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F

__all__ = [
    "NEG_INF", "layer_norm", "linear_col", "linear_row", "split_qkv", "causal_prefix_mask",
    "assign_cache", "attention_core", "attention_forward", "layer_forward", "stack_forward",
    "create_cache", "init_layer_params", "init_stack_params", "uniform_slice",
    "grid_slice_batch_and_sequence", "terapipe_forward_backward", "unsliced_forward_backward",
    "gelu_erf", "LAYER_PARAM_NAMES", "embedding", "vocab_cross_entropy",
]

# transformer_models.py:16 -- fp16 lowest, used as the additive mask value.
NEG_INF = -65504

LAYER_PARAM_NAMES = (
    "attn_ln.weight", "attn_ln.bias",
    "attn.in_proj.weight", "attn.in_proj.bias",
    "attn.out_proj.weight", "attn.out_proj.bias",
    "fc_ln.weight", "fc_ln.bias",
    "fc1.weight", "fc1.bias",
    "fc2.weight", "fc2.bias",
)


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float = 1e-5):
    """nn.LayerNorm(E) as constructed at transformer_models.py:323,325 (torch default eps 1e-5,
    biased variance over the last dimension, affine)."""
    mean = x.mean(dim=-1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * weight + bias


def linear_col(x, weight, bias):
    """mpu.ColumnParallelLinear.forward at tensor-parallel size 1 (mpu/layers.py:252-262):
    identity copy (mpu/mappings.py:26-28) then F.linear(x, W, b) with W stored [out, in]."""
    return torch.matmul(x, weight.t()) + bias


def linear_row(x, weight, bias):
    """mpu.RowParallelLinear.forward at tensor-parallel size 1 (mpu/layers.py:328-353):
    F.linear without bias (:335), identity reduce, then ``+ bias`` as a separate op (:346-347)."""
    y = torch.matmul(x, weight.t())
    return y + bias


def gelu_erf(x):
    """erf-form GeLU; not on the reference path (it uses relu_, transformer_models.py:282) but
    offered by the fused bias+activation kernel, so the oracle states it for that kernel's test."""
    return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))


def split_qkv(qkv: torch.Tensor, num_heads: int):
    """transformer_models.py:217 -- ``in_proj(x).view(T, B*H, 3*Dh).transpose_(0, 1).chunk(3, -1)``.
    Feature j of in_proj belongs to head j // (3*Dh); inside a head the order is [q | k | v]."""
    T, B, E3 = qkv.shape
    Dh = E3 // (3 * num_heads)
    q, k, v = qkv.view(T, B * num_heads, 3 * Dh).transpose(0, 1).chunk(3, dim=-1)
    return q, k, v


def causal_prefix_mask(T: int, P: int, dtype=torch.float32, device=None):
    """transformer_models.py:220,229 -- additive mask [T, P+T]: zeros over the prefix columns,
    NEG_INF strictly above the diagonal of the slice block."""
    tri = torch.full((T, T), NEG_INF, dtype=dtype, device=device).triu_(1)
    if P > 0:
        return torch.cat([torch.zeros(T, P, dtype=dtype, device=device), tri], dim=1)
    return tri


class _AssignCache(torch.autograd.Function):
    """transformer_models.py:177-193.  Forward writes ``value`` into ``cache[:, P:S, :]`` in place
    (through .data, no version bump) and returns the cache.  Backward hands the slice rows of the
    incoming gradient to ``value`` and a clone with those rows zeroed to ``cache``."""

    @staticmethod
    def forward(ctx, cache, value, lo, hi):
        ctx.lo, ctx.hi = lo, hi
        cache.data[:, lo:hi, :] = value
        return cache

    @staticmethod
    def backward(ctx, g):
        grad_value = g[:, ctx.lo:ctx.hi, :]
        grad_cache = g.clone()
        grad_cache.data[:, ctx.lo:ctx.hi, :] = 0
        return grad_cache, grad_value, None, None


def assign_cache(cache, value, lo, hi):
    return _AssignCache.apply(cache, value, lo, hi)


def attention_core(q, k, v, mask, T, B):
    """attn_helper, transformer_models.py:235-245: bmm(q, k^T) + mask -> softmax in fp32 (or the
    input dtype if wider) -> bmm(P, v) -> [T, B, E] with heads concatenated in order."""
    w = torch.bmm(q, k.transpose(1, 2))
    w = w + mask[None, :, :]
    sm_dtype = torch.float64 if w.dtype == torch.float64 else torch.float32
    p = F.softmax(w, dim=-1, dtype=sm_dtype).type_as(w)
    a = torch.bmm(p, v)
    return a.transpose(0, 1).contiguous().view(T, B, -1)


def attention_forward(p: Dict[str, torch.Tensor], prefix: str, x, num_heads: int,
                      full_cache=None, cache_len: int = 0):
    """MultiheadLMAttentionWithCache.forward, transformer_models.py:214-255."""
    T, B, E = x.shape
    Dh = E // num_heads
    assert Dh * num_heads == E                                      # :209-211
    scaling = Dh ** -0.5                                            # :212
    qkv = linear_col(x, p[prefix + "in_proj.weight"], p[prefix + "in_proj.bias"])
    q, new_k, new_v = split_qkv(qkv, num_heads)                     # :217
    q = q * scaling                                                 # :219
    if full_cache is not None:
        S = cache_len + T                                           # :222
        cache_k, cache_v = full_cache
        cache_k = assign_cache(cache_k, new_k, cache_len, S)        # :225
        cache_v = assign_cache(cache_v, new_v, cache_len, S)        # :226
        k = cache_k[:, :S, :]                                       # :227
        v = cache_v[:, :S, :]                                       # :228
        mask = causal_prefix_mask(T, cache_len, x.dtype, x.device)  # :229
    else:
        assert cache_len == 0                                       # :231
        k, v = new_k, new_v
        mask = causal_prefix_mask(T, 0, x.dtype, x.device)
    a = attention_core(q, k, v, mask, T, B)
    out = linear_row(a, p[prefix + "out_proj.weight"], p[prefix + "out_proj.bias"])  # :251
    if full_cache is not None:
        return out, (cache_k, cache_v)
    return out, None


def layer_forward(p: Dict[str, torch.Tensor], x, num_heads: int, full_cache=None,
                  cache_len: int = 0, prefix: str = "", activation: str = "relu", relu_mask=None,
                  preact_sink: Optional[list] = None):
    """TransformerLayer.forward, transformer_models.py:273-285 (pre-LN block, ReLU MLP).

    relu_mask (optional bool tensor shaped like the fc1 output) replaces ``z > 0`` as the ReLU's
    active set: a 16-bit run decides the sign of near-zero pre-activations by its own rounding, and a
    parity test that wants to measure arithmetic error rather than those sign flips hands the mask of
    the run under test to the oracle.  The reference path is relu_mask=None.
    preact_sink (optional list) receives a detached copy of the fc1 output before the activation, so that a
    test can check the active set it hands in against the sign of the oracle's own pre-activations."""
    y = x
    h = layer_norm(x, p[prefix + "attn_ln.weight"], p[prefix + "attn_ln.bias"])       # :275
    h, new_cache = attention_forward(p, prefix + "attn.", h, num_heads, full_cache, cache_len)
    h = h + y                                                                        # :277
    y = h
    z = layer_norm(h, p[prefix + "fc_ln.weight"], p[prefix + "fc_ln.bias"])           # :280
    z = linear_col(z, p[prefix + "fc1.weight"], p[prefix + "fc1.bias"])
    if preact_sink is not None:
        preact_sink.append(z.detach().clone())
    if activation == "relu":
        z = torch.relu(z) if relu_mask is None else z * relu_mask.to(z.dtype)        # :282
    else:
        z = gelu_erf(z)
    z = linear_row(z, p[prefix + "fc2.weight"], p[prefix + "fc2.bias"])               # :283
    return z + y, new_cache                                                          # :284-285


def stack_forward(params: List[Dict[str, torch.Tensor]], x, num_heads: int, cache, cache_len: int,
                  activation: str = "relu", relu_masks=None, preact_sink: Optional[list] = None):
    """TransformerLayers.forward, terapipe.py:79-86; cache is the flat list [k0, v0, k1, v1, ...].
    relu_masks: optional list (one per layer) passed to layer_forward; preact_sink: optional list that
    receives every layer's fc1 pre-activation in layer order."""
    cache_outputs = []
    for i, p in enumerate(params):
        x, (ko, vo) = layer_forward(p, x, num_heads, (cache[2 * i], cache[2 * i + 1]), cache_len,
                                    activation=activation,
                                    relu_mask=None if relu_masks is None else relu_masks[i],
                                    preact_sink=preact_sink)
        cache_outputs += [ko, vo]
    return x, cache_outputs


def create_cache(n_layers: int, batch_size: int, num_heads: int, seq_len: int, head_dim: int,
                 dtype=torch.float32, device=None):
    """TransformerLayers.create_cache (terapipe.py:70-77) over create_attn_cache
    (transformer_models.py:257-261): zeros [B*H, L, Dh] for K and V of every layer."""
    cache = []
    for _ in range(n_layers):
        cache += [torch.zeros(batch_size * num_heads, seq_len, head_dim, dtype=dtype, device=device),
                  torch.zeros(batch_size * num_heads, seq_len, head_dim, dtype=dtype, device=device)]
    return cache


def init_layer_params(E: int, Fdim: int, std: float = 0.02, dtype=torch.float32,
                      generator: Optional[torch.Generator] = None) -> Dict[str, torch.Tensor]:
    """Synthetic weights of the benchmark configs: W ~ N(0, std), biases 0 (mpu/layers.py:240-241,
    :316-317), LayerNorm gamma 1 / beta 0."""
    def w(*shape):
        return (torch.randn(*shape, generator=generator, dtype=torch.float32) * std).to(dtype)
    return {
        "attn_ln.weight": torch.ones(E, dtype=dtype), "attn_ln.bias": torch.zeros(E, dtype=dtype),
        "attn.in_proj.weight": w(3 * E, E), "attn.in_proj.bias": torch.zeros(3 * E, dtype=dtype),
        "attn.out_proj.weight": w(E, E), "attn.out_proj.bias": torch.zeros(E, dtype=dtype),
        "fc_ln.weight": torch.ones(E, dtype=dtype), "fc_ln.bias": torch.zeros(E, dtype=dtype),
        "fc1.weight": w(Fdim, E), "fc1.bias": torch.zeros(Fdim, dtype=dtype),
        "fc2.weight": w(E, Fdim), "fc2.bias": torch.zeros(E, dtype=dtype),
    }


def init_stack_params(n_layers, E, Fdim, std=0.02, dtype=torch.float32, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [init_layer_params(E, Fdim, std, dtype, g) for _ in range(n_layers)]


def embedding(ids, weight):
    """VocabParallelEmbedding.forward at tensor-parallel size 1 (mpu/layers.py:126-141): ids outside the
    partition's vocabulary range [0, V) are looked up as row 0 and their output rows zeroed; the all-reduce
    is the identity.  Pinned by F.embedding and a Python loop (tests/test_oracle_pins.py)."""
    V = weight.shape[0]
    mask = (ids < 0) | (ids >= V)
    masked = ids.clone()
    masked[mask] = 0
    out = weight[masked]                                                             # F.embedding, :134-137
    out = torch.where(mask.unsqueeze(-1), torch.zeros((), dtype=out.dtype), out)     # :139
    return out


def vocab_cross_entropy(logits, target):
    """_VocabParallelCrossEntropy.forward at tensor-parallel size 1 (mpu/cross_entropy.py:25-77), without
    the in-place overwrites: per-token loss = log(sum exp(logits - max)) - (logits - max)[target].
    Pinned by F.cross_entropy(reduction='none') and a Python loop."""
    z = logits - logits.max(dim=-1, keepdim=True)[0]                                 # :28-33
    predicted = z.gather(-1, target.unsqueeze(-1)).squeeze(-1)                       # :48-57
    return torch.log(torch.exp(z).sum(dim=-1)) - predicted                           # :63-71


def uniform_slice(length: int, n_slices: int) -> List[int]:
    """utils.py:110-111 -- the first ``length % n`` slices get one extra element."""
    return [length // n_slices + int(i < length % n_slices) for i in range(n_slices)]


def grid_slice_batch_and_sequence(x, batch_slices, seq_slices, requires_grad=False,
                                  batch_dim=1, sequence_dim=0):
    """transformer_models.py:393-409 -- object ndarray [n_batch_slices, n_seq_slices] of detached,
    contiguous leaf copies."""
    out = np.empty((len(batch_slices), len(seq_slices)), dtype="O")
    b0 = 0
    for i, bs in enumerate(batch_slices):
        s0 = 0
        for j, ss in enumerate(seq_slices):
            piece = x.narrow(sequence_dim, s0, ss).narrow(batch_dim, b0, bs)
            out[i, j] = piece.detach().contiguous().requires_grad_(requires_grad)
            s0 += ss
        assert s0 == x.size(sequence_dim)
        b0 += bs
    assert b0 == x.size(batch_dim)
    return out


def terapipe_forward_backward(params: List[Dict[str, torch.Tensor]], x, dy, num_heads: int,
                              batch_slices: Sequence[int], seq_slices: Sequence[int],
                              return_cache_grads: bool = False, activation: str = "relu", relu_masks=None,
                              preacts: Optional[dict] = None):
    """TeraPipe.forward (terapipe.py:238-271) followed by TeraPipeBackwardPassHook.backward
    (terapipe.py:167-201) on a single pipeline stage.

    ``params`` must be leaf tensors with requires_grad=True; their .grad accumulates over slices
    exactly as in the reference (autograd sum).  Returns (y, dx, final_caches[, cache_grads]) where
    final_caches[b] is the flat K/V list after the last slice of batch slice b and cache_grads[b][i]
    is the list of .grad tensors of the cache inputs of slice i.  relu_masks, if given, maps
    (batch slice, sequence slice) to the per-layer list of ReLU active sets (see layer_forward);
    preacts, if given, is filled with (batch slice, sequence slice) -> per-layer fc1 pre-activations.
    """
    L = x.size(0)
    E = x.size(2)
    Dh = E // num_heads
    n_layers = len(params)
    inputs = grid_slice_batch_and_sequence(x, batch_slices, seq_slices, requires_grad=True)
    nb, ns = len(batch_slices), len(seq_slices)
    cache_inputs = np.empty((nb, ns), dtype="O")
    cache_outputs = np.empty((nb, ns), dtype="O")
    outputs = np.empty((nb, ns), dtype="O")
    final_caches = []
    for b in range(nb):
        cache = create_cache(n_layers, inputs[b, 0].size(1), num_heads, L, Dh, x.dtype, x.device)  # :251
        cache_len = 0
        for i in range(ns):
            xi = inputs[b, i]
            cache = [c.detach().requires_grad_() for c in cache]                          # :257
            sink = None
            if preacts is not None:
                sink = preacts[(b, i)] = []
            y, cache_out = stack_forward(params, xi, num_heads, cache, cache_len, activation,      # :258
                                         None if relu_masks is None else relu_masks[(b, i)], sink)
            cache_inputs[b, i] = cache
            cache_outputs[b, i] = cache_out
            cache = cache_out
            outputs[b, i] = y
            cache_len += xi.size(0)                                                       # :264
        final_caches.append([c.detach().clone() for c in cache])
    y_full = torch.cat([torch.cat(list(outputs[b]), dim=0) for b in range(nb)], dim=1).detach()  # :206-207

    grad_outputs = grid_slice_batch_and_sequence(dy, batch_slices, seq_slices)             # :171-174
    for b in reversed(range(nb)):
        da = []
        for i in reversed(range(ns)):
            a = list(cache_outputs[b, i]) if i < ns - 1 else []                            # :186-189
            torch.autograd.backward([outputs[b, i]] + a, [grad_outputs[b, i]] + da)        # :190
            da = [t.grad for t in cache_inputs[b, i]]                                      # :191
    dx = torch.cat([torch.cat([inputs[b, i].grad for i in range(ns)], dim=0) for b in range(nb)], dim=1)
    if return_cache_grads:
        cg = [[[t.grad for t in cache_inputs[b, i]] for i in range(ns)] for b in range(nb)]
        return y_full, dx, final_caches, cg
    return y_full, dx, final_caches


def unsliced_forward_backward(params, x, dy, num_heads):
    """One slice covering the whole batch and sequence: the comparison run of
    NCCLTransformerRunner.verify (test_transformer_terapipe.py:347-348).  Uses plain causal
    self-attention without a cache (full_cache=None path, transformer_models.py:230-234)."""
    xi = x.detach().clone().requires_grad_(True)
    h = xi
    for p in params:
        h, _ = layer_forward(p, h, num_heads, None, 0)
    h.backward(dy)
    return h.detach(), xi.grad
