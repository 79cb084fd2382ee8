"""Host-side mirror of the reference's sliced runner (terapipe.py of the reference) on one GPU:
``TransformerLayers`` (terapipe.py:52-95) and ``TeraPipe`` (terapipe.py:219-271) with the reverse-order
slice backward of ``TeraPipeBackwardPassHook`` (terapipe.py:154-212).

``TeraPipe.forward`` runs the whole slice grid inside ONE autograd node.  Its backward walks the slices
in reverse, hands dK/dV of the prefix rows from slice i+1 to slice i through persistent fp32 gradient
caches (instead of a full-length clone per slice, reference transformer_models.py:188), and can defer
the weight-gradient GEMMs to one GEMM per weight over all tokens (dW = dY_all^T X_all equals the sum
over slices of dY_i^T X_i).  Pipeline send/recv, process groups and the optimizer are not part of
this path.
"""
import numpy as np
import torch
import torch.nn as nn

from . import _layer_core as core
from . import ops
from ._lib import TP_EPI_STORE, TP_GEMM_TN
from .transformer_models import ModelParallelTransformerLayer, grid_slice_batch_and_sequence


def loss_func(y):
    """Reference terapipe.py:48-49."""
    return torch.mean(y)


def uniform_slice(length, n_slices):
    """Reference utils.py:110-111."""
    return [length // n_slices + int(i < length % n_slices) for i in range(n_slices)]


class TransformerLayers(nn.Module):
    """Reference terapipe.py:52-95.  mixed_precision selects fp16 as the reference does
    (``layer.half()``, terapipe.py:67); ``dtype`` overrides it (bf16 for the 175B/44B shapes)."""

    def __init__(self, n_layers, embedding_dim, ffn_embedding_dim, num_attention_heads, mixed_precision=True,
                 dtype=None, device="cuda", activation="relu"):
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


class _TeraPipeFunction(torch.autograd.Function):
    """forward: every (batch slice, sequence slice) through the whole layer stack, slice-major.
    backward: reverse-order slices (terapipe.py:182-191 of the reference)."""

    @staticmethod
    def forward(ctx, runner, inputs, *flat_params):
        layers = runner.layers
        n_layers = layers.n_layers
        heads = layers.num_attention_heads
        ws = [dict(zip(core.PARAM_NAMES, flat_params[12 * i:12 * i + 12])) for i in range(n_layers)]
        act = [l.activation for l in layers.layers]
        need_state = any(ctx.needs_input_grad)
        xs = grid_slice_batch_and_sequence(inputs, runner.batch_slices, runner.seq_slices, requires_grad=False,
                                           batch_dim=runner.batch_dim, sequence_dim=runner.sequence_dim)
        nb, ns = len(runner.batch_slices), len(runner.seq_slices)
        states = np.empty((nb, ns), dtype="O")
        outs = np.empty((nb, ns), dtype="O")
        caches = []
        for b in range(nb):
            cache = layers.create_cache(runner.batch_slices[b], runner.seq_len)      # terapipe.py:251
            cache_len = 0
            for i in range(ns):
                x = xs[b, i]
                sts = []
                for l in range(n_layers):
                    x, st = core.layer_fwd(ws[l], x, heads, cache[2 * l], cache[2 * l + 1], cache_len, act[l],
                                           need_state=need_state)
                    sts.append(st)
                states[b, i] = sts
                outs[b, i] = x
                cache_len += runner.seq_slices[i]                                    # terapipe.py:264
            caches.append(cache)
        runner.last_caches = caches
        if runner.keep_states:
            runner.last_states = states.copy()
        y = torch.cat([torch.cat(list(outs[b]), dim=runner.sequence_dim) for b in range(nb)], dim=runner.batch_dim)
        ctx.runner, ctx.ws, ctx.act, ctx.states = runner, ws, act, states
        ctx.in_shape = inputs.shape
        return y

    @staticmethod
    def backward(ctx, grad_y):
        runner, ws, act, states = ctx.runner, ctx.ws, ctx.act, ctx.states
        layers = runner.layers
        n_layers, heads = layers.n_layers, layers.num_attention_heads
        E, F = layers.embedding_dim, layers.ffn_embedding_dim
        Dh = E // heads
        dev, dt = grad_y.device, grad_y.dtype
        nb, ns = len(runner.batch_slices), len(runner.seq_slices)
        dys = grid_slice_batch_and_sequence(grad_y, runner.batch_slices, runner.seq_slices,
                                            batch_dim=runner.batch_dim, sequence_dim=runner.sequence_dim)
        gdt = torch.float32 if runner.fp32_grad_cache else dt
        nsmall = core.small_acc_numel(E, F)
        small = torch.zeros(n_layers, nsmall, dtype=torch.float32, device=dev)
        small_views = [core.small_acc_views(small[l], E, F) for l in range(n_layers)]
        wgrads = [{n: torch.empty_like(ws[l][n]) for n in core.BIG_PARAMS} for l in range(n_layers)]
        defer = runner.defer_weight_grads
        stash = [[{n: [] for n in core.BIG_PARAMS} for _ in range(n_layers)]] if defer else None
        dxs = np.empty((nb, ns), dtype="O")
        first = True
        for b in reversed(range(nb)):
            Bs = runner.batch_slices[b]
            # gradient caches of this batch slice: every row is written (=) before it is read (+=),
            # because the last slice covers all rows, so no zero fill is needed
            gks = [torch.empty(Bs * heads, runner.seq_len, Dh, dtype=gdt, device=dev) for _ in range(2 * n_layers)]
            for i in reversed(range(ns)):
                last = i == ns - 1
                dx = dys[b, i]
                for l in reversed(range(n_layers)):
                    d = {} if defer else None
                    dx = core.layer_bwd(ws[l], states[b, i][l], dx, heads, gks[2 * l], gks[2 * l + 1], wgrads[l],
                                        not first, small_views[l], accumulate_prefix=not last,
                                        has_incoming=not last, zero_slice_rows=False, activation=act[l], defer=d)
                    if defer:
                        for n in core.BIG_PARAMS:
                            stash[0][l][n].append(d[n])
                states[b, i] = None
                dxs[b, i] = dx
                first = False
        if defer:
            for l in range(n_layers):
                for n in core.BIG_PARAMS:
                    pairs = stash[0][l][n]
                    dY = torch.cat([p[0] for p in pairs], dim=0)
                    X = torch.cat([p[1] for p in pairs], dim=0)
                    ops.gemm(TP_GEMM_TN, dY, X, dY.shape[1], X.shape[1], dY.shape[0], C=wgrads[l][n],
                             epilogue=TP_EPI_STORE)
        grads = []
        for l in range(n_layers):
            g = dict(wgrads[l])
            for n in core.SMALL_PARAMS:
                t = torch.empty_like(ws[l][n])
                ops.accum_cast(t, small_views[l][n], False)
                g[n] = t
            grads += [g[n] for n in core.PARAM_NAMES]
        dinputs = None
        if ctx.needs_input_grad[1]:
            dinputs = torch.cat([torch.cat(list(dxs[b]), dim=runner.sequence_dim) for b in range(nb)],
                                dim=runner.batch_dim)
        ctx.states = None
        return (None, dinputs) + tuple(grads)


class TeraPipe(nn.Module):
    """Reference terapipe.py:219-271 on a single stage.  ``forward(inputs)`` returns the concatenated
    outputs [seq_len, batch, E]; ``loss(y).backward()`` then runs the reverse-order slice backward and
    leaves the summed-over-slices gradients in the layers' parameters (and in ``inputs.grad`` when the
    input requires grad).

    defer_weight_grads: run one weight-gradient GEMM per weight over all tokens instead of one per slice.
    fp32_grad_cache: keep the cross-slice dK/dV accumulators in fp32 (one rounding at the end) instead of
    the cache dtype the reference uses.
    """

    def __init__(self, layers, batch_size, seq_len, batch_slices, seq_slices, batch_dim=1, sequence_dim=0,
                 defer_weight_grads=True, fp32_grad_cache=True):
        super().__init__()
        assert sum(batch_slices) == batch_size and sum(seq_slices) == seq_len
        assert batch_dim == 1 and sequence_dim == 0, "layers take [seq, batch, embed] inputs"
        self.batch_size, self.seq_len = batch_size, seq_len
        self.batch_slices, self.seq_slices = list(batch_slices), list(seq_slices)
        self.batch_dim, self.sequence_dim = batch_dim, sequence_dim
        self.layers = layers
        self.defer_weight_grads = defer_weight_grads
        self.fp32_grad_cache = fp32_grad_cache
        self.last_caches = None
        self.keep_states = False   # debugging / tests: keep the per-slice saved activations of the last forward
        self.last_states = None

    @property
    def n_batch_slices(self):
        return len(self.batch_slices)

    @property
    def n_input_slices(self):
        return len(self.seq_slices)

    def forward(self, inputs=None):
        if inputs is None:
            inputs = self.layers.create_inputs(self.batch_size, self.seq_len)
        assert inputs.size(self.sequence_dim) == self.seq_len and inputs.size(self.batch_dim) == self.batch_size
        flat = []
        for layer in self.layers.layers:
            p = layer.param_dict()
            flat += [p[n] for n in core.PARAM_NAMES]
        return _TeraPipeFunction.apply(self, inputs, *flat)
