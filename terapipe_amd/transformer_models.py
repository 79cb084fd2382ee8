"""Host-side mirror of the reference's layer call surface (transformer_models.py of the reference):
same class names, constructor arguments, state-dict keys, forward signatures and assertion behaviour,
with the arithmetic done by the HIP kernels of libterapipe_hip.so.

Differences that are deliberate: no ``mpu`` / ``torch.distributed`` process group is needed (tensor-
parallel size is 1, mpu/mappings.py:26-28 of the reference makes every collective an identity there);
the head dimension is one of 16, 32, 64, 80, 96, 128 (every entry of MODEL_CONFIGS); the K/V caches are written by the QKV GEMM's epilogue rather than by
a separate _AssignCache op, with the same in-place, alias-returning semantics and the same gradient
contract (reference transformer_models.py:177-193).
"""
import warnings

import numpy as np
import torch
import torch.nn as nn

from . import _layer_core as core
from . import ops
from ._lib import TP_EPI_ACCUMULATE, TP_EPI_BIAS, TP_EPI_STORE, TP_GEMM_NN, TP_GEMM_NT, TP_GEMM_TN

# reference transformer_models.py:16 -- kept for callers that import it; the kernels mask by index.
NEG_INF = -65504

# name -> (n_layers, hidden_size, sequence_length, num_attention_heads); reference transformer_models.py:17-59
MODEL_CONFIGS = {
    "test": (24, 256, 128, 4),
    "test-l512": (512, 256, 128, 4),
    "test-s1024": (48, 2048, 1024, 32),
    "test-s2048": (48, 2048, 2048, 32),
    "test-h3072": (48, 3072, 2048, 48),
    "gpt2-1hm": (12, 768, 1024, 12),
    "gpt2-3hm": (24, 1024, 1024, 16),
    "gpt2-7hm": (36, 1280, 1024, 20),
    "gpt2-1b": (48, 1600, 1024, 25),
    "megatron-1b": (40, 1536, 1024, 16),
    "megatron-2b": (54, 1920, 1024, 20),
    "megatron-4b": (64, 2304, 1024, 24),
    "megatron-8b": (72, 3072, 1024, 32),
    "gpt3-1hm": (12, 768, 2048, 12),
    "gpt3-3hm": (24, 1024, 2048, 16),
    "gpt3-7hm": (24, 1536, 2048, 16),
    "gpt3-1b": (24, 2048, 2048, 16),
    "gpt3-2b": (32, 2560, 2048, 32),
    "gpt3-6b": (32, 4096, 2048, 32),
    "gpt3-13b": (40, 5120, 2048, 40),
    "gpt3-44b": (96, 6144, 2048, 48),
    "gpt3-175b": (96, 12288, 2048, 96),
    "gpt3-13b-4096": (40, 5120, 4096, 40),
    "gpt3-13b-6144": (40, 5120, 6144, 40),
    "gpt3-13b-8192": (40, 5120, 8192, 40),
    "gpt3-175b-megatron": (48, 6144, 2048, 384),
    "gpt2-1hm-single-device": (10, 768, 2048, 12),
    "gpt2-3hm-single-device": (8, 1024, 2048, 16),
    "gpt2-7hm-single-device": (6, 1280, 2048, 20),
    "gpt2-1b-single-device": (4, 1600, 2048, 25),
    "gpt3-1b-single-device": (5, 2048, 2048, 16),
    "gpt3-2b-single-device": (3, 2560, 2048, 32),
    "gpt3-6b-single-device": (2, 4096, 2048, 32),
    "gpt3-13b-single-device": (1, 5120, 2048, 40),
    "gpt3-175b-single-node": (2, 12288, 2048, 96),
}

# reference transformer_models.py:61-69
BATCH_CONFIGS = {"gpt3-1b": 72, "gpt3-13b": 32, "gpt3-44b": 16, "gpt3-175b": 2,
                 "gpt3-13b-4096": 8, "gpt3-13b-6144": 4, "gpt3-13b-8192": 2}


class TransformerConfig:
    """Shape bookkeeping of reference transformer_models.py:71-174 (single device: no placement)."""

    def __init__(self, batch_size=1, seq_len=1024, n_layers=12, embedding_dim=768, ffn_embedding_dim=None,
                 num_attention_heads=None, model_name=None):
        self.batch_size = batch_size
        if model_name is None:
            self.seq_len, self.n_layers, self.embedding_dim = seq_len, n_layers, embedding_dim
            self.ffn_embedding_dim = ffn_embedding_dim if ffn_embedding_dim else embedding_dim * 4
            self.num_attention_heads = num_attention_heads if num_attention_heads else embedding_dim // 64
        else:
            self.n_layers, self.embedding_dim, self.seq_len, self.num_attention_heads = MODEL_CONFIGS[model_name]
            self.ffn_embedding_dim = self.embedding_dim * 4

    @classmethod
    def from_predefined_model(cls, model_name, batch_size=1):
        return cls(batch_size=batch_size, model_name=model_name)

    @property
    def attention_heads_dim(self):
        return self.embedding_dim // self.num_attention_heads


# ------------------------------------------------------------------------------------------------
# linear layers (mpu/layers.py:193-353 of the reference at tensor-parallel size 1)
# ------------------------------------------------------------------------------------------------
class _LinearFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias):
        lead = x.shape[:-1]
        x2d = x.reshape(-1, x.shape[-1]).contiguous()
        M, K = x2d.shape
        N = weight.shape[0]
        y = torch.empty(M, N, dtype=x.dtype, device=x.device)
        if bias is not None:
            ops.gemm(TP_GEMM_NT, x2d, weight, M, N, K, C=y, epilogue=TP_EPI_BIAS, bias=bias)
        else:
            ops.gemm(TP_GEMM_NT, x2d, weight, M, N, K, C=y, epilogue=TP_EPI_STORE)
        ctx.save_for_backward(x2d, weight)
        ctx.has_bias = bias is not None
        ctx.lead = lead
        return y.view(*lead, N)

    @staticmethod
    def backward(ctx, dy):
        x2d, weight = ctx.saved_tensors
        M, K = x2d.shape
        N = weight.shape[0]
        dy2d = dy.reshape(M, N).contiguous()
        dx = torch.empty_like(x2d)
        ops.gemm(TP_GEMM_NN, dy2d, weight, M, K, N, C=dx)
        dw = torch.empty_like(weight)
        ops.gemm(TP_GEMM_TN, dy2d, x2d, N, K, M, C=dw)
        db = None
        if ctx.has_bias:
            acc = torch.zeros(N, dtype=torch.float32, device=dy.device)
            ops.colsum_acc(dy2d, acc)
            db = torch.empty(N, dtype=weight.dtype, device=dy.device)
            ops.accum_cast(db, acc, False)
        return dx.view(*ctx.lead, K), dw, db


class _ParallelLinearBase(nn.Module):
    def __init__(self, input_size, output_size, bias=True, init_method=nn.init.xavier_normal_, device="cuda"):
        super().__init__()
        self.input_size, self.output_size = input_size, output_size
        self.weight = nn.Parameter(torch.empty(output_size, input_size, device=device))   # [out, in]
        init_method(self.weight)
        if bias:
            self.bias = nn.Parameter(torch.zeros(output_size, device=device))              # always zero-init
        else:
            self.register_parameter("bias", None)

    def forward(self, input_):
        return _LinearFunction.apply(input_, self.weight, self.bias)


class ColumnParallelLinear(_ParallelLinearBase):
    """mpu.ColumnParallelLinear (reference mpu/layers.py:193-262) at tensor-parallel size 1:
    Y = X W^T + b, W stored [out, in], bias zero-initialised."""

    def __init__(self, input_size, output_size, bias=True, gather_output=True,
                 init_method=nn.init.xavier_normal_, device="cuda"):
        super().__init__(input_size, output_size, bias, init_method, device)
        self.gather_output = gather_output


class RowParallelLinear(_ParallelLinearBase):
    """mpu.RowParallelLinear (reference mpu/layers.py:265-353) at tensor-parallel size 1."""

    def __init__(self, input_size, output_size, bias=True, input_is_parallel=False,
                 init_method=nn.init.xavier_normal_, device="cuda"):
        super().__init__(input_size, output_size, bias, init_method, device)
        self.input_is_parallel = input_is_parallel


# ------------------------------------------------------------------------------------------------
# attention module and layer
# ------------------------------------------------------------------------------------------------
def _check_cache(full_cache, B, H, Dh, S, dtype):
    k, v = full_cache
    for c in (k, v):
        assert c.dim() == 3 and c.shape[0] == B * H and c.shape[2] == Dh, \
            "cache must be [batch*heads, seq_len, head_dim]"
        assert c.shape[1] >= S, "cache_len + slice length exceeds the cache"
        assert c.dtype == dtype and c.is_contiguous()
    return k, v


def _temp_cache(B, H, T, Dh, like):
    return (torch.empty(B * H, T, Dh, dtype=like.dtype, device=like.device),
            torch.empty(B * H, T, Dh, dtype=like.dtype, device=like.device))


def _grads_can_go_in_place(w):
    """Every parameter of the layer already has a dense .grad of its own dtype to add to."""
    for p in w.values():
        g = p.grad
        if g is None or g.dtype != p.dtype or g.shape != p.shape or not g.is_contiguous():
            return False
    return True


class _GradOptions:
    """How a layer's backward hands its parameter gradients to autograd (TransformerLayer's two switches) and,
    for deferred weight gradients, the sequences whose backward is under way (keyed by their K cache)."""
    __slots__ = ("in_place", "defer", "pending")

    def __init__(self):
        self.in_place, self.defer, self.pending = False, False, {}


class _PendingGrads:
    """Deferred weight gradients of one sequence in one layer: the output gradients and inputs of the four
    linears for every position whose slice has run its backward (rows [low, rows); the reverse-slice order
    fills them from the end), and the fp32 sums of the vector-parameter gradients so far."""
    __slots__ = ("rows", "low", "dqkv", "dh", "dz1", "dout", "xn", "o", "hn", "a", "acc")

    def __init__(self, rows, E, F, dtype, device):
        new = lambda n: torch.empty(rows, n, dtype=dtype, device=device)
        self.rows = self.low = rows
        self.dqkv, self.dh, self.dz1, self.dout = new(3 * E), new(E), new(F), new(E)
        self.xn, self.o, self.hn, self.a = new(E), new(E), new(E), new(F)
        self.acc = torch.zeros(core.small_acc_numel(E, F), dtype=torch.float32, device=device)


class _LayerFunction(torch.autograd.Function):
    """One whole layer over one slice.  Inputs: x, k_cache, v_cache (or None, None), then the 12
    parameters in core.PARAM_NAMES order.  Outputs: out, and the two caches when given.

    Backward of a slice: the data gradients (core.layer_bwd), then the four weight gradients as one grouped
    library call and the eight vector-parameter gradients as one launch.  opts (_GradOptions):
    in_place -- where every parameter already has a .grad, add the gradients to it inside those launches (the
    GEMM's accumulate epilogue, one rounding) and hand autograd None, instead of returning twelve tensors that
    autograd adds to .grad one elementwise kernel each;
    defer -- keep the slice's dY / X rows and take the weight gradients once per sequence, over all its rows, in
    the backward of the slice at position 0 (the last one the reverse-slice order reaches); the slices before
    it hand autograd None for the parameters."""

    @staticmethod
    def forward(ctx, heads, cache_len, activation, opts, x, k_cache, v_cache, *params):
        w = dict(zip(core.PARAM_NAMES, params))
        T, B, E = x.shape
        Dh = E // heads
        ctx.has_cache = k_cache is not None
        if not ctx.has_cache:
            k_cache, v_cache = _temp_cache(B, heads, T, Dh, x)
        out, st = core.layer_fwd(w, x.contiguous(), heads, k_cache, v_cache, cache_len, activation)
        ctx.st, ctx.w, ctx.heads, ctx.activation = st, w, heads, activation
        ctx.opts = opts
        ctx.set_materialize_grads(False)
        if ctx.has_cache:
            # the caches were written through their raw pointers (as `cache.data[index] = value` does,
            # reference transformer_models.py:183); returning the inputs makes autograd hand back aliases
            return out, k_cache, v_cache
        return out

    @staticmethod
    def backward(ctx, dout, dk_out=None, dv_out=None):
        st, w, heads, opts = ctx.st, ctx.w, ctx.heads, ctx.opts
        E = st.x.shape[1]
        F = w["fc1.weight"].shape[0]
        if dout is None:
            dout = torch.zeros(st.T, st.B, E, dtype=st.x.dtype, device=st.x.device)
        gk = gv = None
        has_incoming = False
        if ctx.has_cache:
            if dk_out is not None:
                # grad_cache_output.clone(), reference transformer_models.py:188
                gk, gv = dk_out.clone(), (dv_out.clone() if dv_out is not None else torch.zeros_like(dk_out))
                has_incoming = True
            else:
                gk, gv = torch.zeros_like(st.k_cache), torch.zeros_like(st.v_cache)
        M, dt, dev = st.T * st.B, st.x.dtype, dout.device
        dout = dout.contiguous()
        dout2d = dout.view(M, E)
        new = lambda n: torch.empty(M, n, dtype=dt, device=dev)
        pend = None
        if opts.defer and ctx.has_cache:
            # rows [r0, r1) of the sequence's position-indexed gradient buffers
            r0, r1 = st.cache_len * st.B, (st.cache_len + st.T) * st.B
            key = st.k_cache.data_ptr()
            pend = opts.pending.get(key)
            if pend is None or pend.low != r1:
                # the last slice of a sequence opens it; an entry that does not end where this slice begins belongs
                # to a sequence whose backward was abandoned or skipped a slice
                if pend is not None and pend.low < pend.rows:
                    warnings.warn("defer_weight_grads: the backward of a sequence stopped at row %d and never reached "
                                  "its first slice; its weight gradients are dropped" % pend.low)
                pend = opts.pending[key] = _PendingGrads(r1, E, F, dt, dev)
            buf = core.Bufs(dz1=pend.dz1[r0:r1], dhn=new(E), dh=pend.dh[r0:r1], dqkv=pend.dqkv[r0:r1], dxn=new(E))
        else:
            buf = core.Bufs(dz1=new(F), dhn=new(E), dh=new(E), dqkv=new(3 * E), dxn=new(E))
        dx = core.layer_bwd(w, st, dout, heads, gk, gv, accumulate_prefix=True, has_incoming=has_incoming,
                            zero_slice_rows=has_incoming, activation=ctx.activation, buf=buf)
        acc = pend.acc if pend is not None else torch.zeros(core.small_acc_numel(E, F), dtype=torch.float32,
                                                            device=dev)
        sv = core.small_acc_views(acc, E, F)
        ops.vec_param_grads([(buf.dqkv, sv["attn.in_proj.bias"]),
                             (buf.dh, sv["attn.out_proj.bias"]),
                             (buf.dz1, sv["fc1.bias"]),
                             (dout2d, sv["fc2.bias"]),
                             (buf.dxn, st.x, st.mean1, st.rstd1, sv["attn_ln.weight"], sv["attn_ln.bias"]),
                             (buf.dhn, st.h, st.mean2, st.rstd2, sv["fc_ln.weight"], sv["fc_ln.bias"])])
        ctx.st = None
        no_param_grads = (None, None, None, None, dx, gk, gv) + (None,) * len(core.PARAM_NAMES)
        if pend is not None:
            pend.dout[r0:r1].copy_(dout2d)
            pend.xn[r0:r1].copy_(st.xn)
            pend.o[r0:r1].copy_(st.o.view(M, E))
            pend.hn[r0:r1].copy_(st.hn)
            pend.a[r0:r1].copy_(st.a)
            pend.low = r0
            if r0 > 0:
                return no_param_grads
            del opts.pending[key]
            K = pend.rows
            pairs = ((pend.dqkv, pend.xn), (pend.dh, pend.o), (pend.dz1, pend.hn), (pend.dout, pend.a))
        else:
            K = M
            pairs = ((buf.dqkv, st.xn), (buf.dh, st.o.view(M, E)), (buf.dz1, st.hn), (dout2d, st.a))
        in_place = opts.in_place and _grads_can_go_in_place(w)
        epi = TP_EPI_ACCUMULATE if in_place else TP_EPI_STORE
        wgrad = {n: (w[n].grad if in_place else torch.empty_like(w[n])) for n in core.BIG_PARAMS}
        ops.gemm_grouped([(TP_GEMM_TN, dy, xin, wgrad[n].shape[0], wgrad[n].shape[1], K, wgrad[n], epi)
                          for n, (dy, xin) in zip(("attn.in_proj.weight", "attn.out_proj.weight", "fc1.weight",
                                                   "fc2.weight"), pairs)])
        if in_place:
            for n in core.SMALL_PARAMS:
                ops.accum_cast(w[n].grad, sv[n], True)
            return no_param_grads
        flat = torch.empty(acc.numel(), dtype=dt, device=dev)
        ops.accum_cast(flat, acc, False)
        grads = core.small_acc_views(flat, E, F)
        grads.update(wgrad)
        return no_param_grads[:7] + tuple(grads[n] for n in core.PARAM_NAMES)


class _AttentionFunction(torch.autograd.Function):
    """MultiheadLMAttentionWithCache alone: in_proj, cached attention, out_proj (+ bias)."""

    @staticmethod
    def forward(ctx, heads, cache_len, x, k_cache, v_cache, w_in, b_in, w_out, b_out):
        T, B, E = x.shape
        Dh = E // heads
        ctx.has_cache = k_cache is not None
        if not ctx.has_cache:
            k_cache, v_cache = _temp_cache(B, heads, T, Dh, x)
        w = {"attn.in_proj.weight": w_in, "attn.in_proj.bias": b_in}
        x2d = x.contiguous().view(T * B, E)
        q, o, lse = core.attention_fwd(w, x2d, T, B, heads, k_cache, v_cache, cache_len)
        y = torch.empty(T * B, E, dtype=x.dtype, device=x.device)
        ops.gemm(TP_GEMM_NT, o.view(T * B, E), w_out, T * B, E, E, C=y, epilogue=TP_EPI_BIAS, bias=b_out)
        ctx.saved = (x2d, q, o, lse, k_cache, v_cache, w_in, w_out)
        ctx.geom = (heads, cache_len, T, B, E, Dh)
        ctx.set_materialize_grads(False)
        if ctx.has_cache:
            return y.view(T, B, E), k_cache, v_cache
        return y.view(T, B, E)

    @staticmethod
    def backward(ctx, dy, dk_out=None, dv_out=None):
        x2d, q, o, lse, k_cache, v_cache, w_in, w_out = ctx.saved
        heads, cache_len, T, B, E, Dh = ctx.geom
        M = T * B
        if dy is None:
            dy = torch.zeros(T, B, E, dtype=x2d.dtype, device=x2d.device)
        dy2d = dy.contiguous().view(M, E)
        gk = gv = None
        has_incoming = False
        if ctx.has_cache:
            if dk_out is not None:
                gk, gv = dk_out.clone(), (dv_out.clone() if dv_out is not None else torch.zeros_like(dk_out))
                has_incoming = True
            else:
                gk, gv = torch.zeros_like(k_cache), torch.zeros_like(v_cache)
        acc = torch.zeros(4 * E, dtype=torch.float32, device=dy.device)
        acc_in, acc_out = acc[:3 * E], acc[3 * E:]
        d_o = torch.empty(M, E, dtype=dy.dtype, device=dy.device)
        ops.gemm(TP_GEMM_NN, dy2d, w_out, M, E, E, C=d_o)
        dw_out = torch.empty_like(w_out)
        ops.gemm(TP_GEMM_TN, dy2d, o.view(M, E), E, E, M, C=dw_out)
        ops.colsum_acc(dy2d, acc_out)
        dqkv = torch.empty(M, 3 * E, dtype=dy.dtype, device=dy.device)
        ops.attn_prefix_bwd(q, k_cache, v_cache, o, lse, d_o, dqkv, gk, gv, B, heads, Dh, T, cache_len,
                            float(Dh) ** -0.5, True, has_incoming, has_incoming, colsum_dqkv_acc=acc_in)
        dx = torch.empty(M, E, dtype=dy.dtype, device=dy.device)
        ops.gemm(TP_GEMM_NN, dqkv, w_in, M, E, 3 * E, C=dx)
        dw_in = torch.empty_like(w_in)
        ops.gemm(TP_GEMM_TN, dqkv, x2d, 3 * E, E, M, C=dw_in)
        db_in = torch.empty(3 * E, dtype=w_in.dtype, device=dy.device)
        db_out = torch.empty(E, dtype=w_in.dtype, device=dy.device)
        ops.accum_cast(db_in, acc_in, False)
        ops.accum_cast(db_out, acc_out, False)
        ctx.saved = None
        return None, None, dx.view(T, B, E), gk, gv, dw_in, db_in, dw_out, db_out


class MultiheadLMAttentionWithCache(nn.Module):
    """Reference transformer_models.py:196-261.  forward(x, full_cache=None, cache_len=0) returns
    (attn_out [T, B, E], (cache_k, cache_v) | None); the caches are updated in place on rows
    [cache_len, cache_len + T)."""

    def __init__(self, embed_dim, num_heads, bias=True, device="cpu"):
        super().__init__()
        self.embed_dim = embed_dim
        self.in_proj = ColumnParallelLinear(embed_dim, 3 * embed_dim, bias=bias, gather_output=False, device=device)
        self.out_proj = RowParallelLinear(embed_dim, embed_dim, bias=bias, input_is_parallel=True, device=device)
        if not bias:
            # the projection kernels fuse a bias: without one (reference transformer_models.py:197, :202-203)
            # they are given zeros, which are no parameters and appear in no state dict
            self.register_buffer("_no_in_bias", torch.zeros(3 * embed_dim, device=device), persistent=False)
            self.register_buffer("_no_out_bias", torch.zeros(embed_dim, device=device), persistent=False)
        self.num_heads = num_heads
        self.head_dim = embed_dim // num_heads
        assert self.head_dim * num_heads == self.embed_dim, "embed_dim must be divisible by num_heads"
        self.scaling = self.head_dim ** -0.5

    def forward(self, x, full_cache=None, cache_len=0, checkpoint_gradients=False):
        # checkpoint_gradients (reference checkpoint.py:24-43) needs no separate path: the attention
        # backward always recomputes the probabilities from q, k and the saved log-sum-exp.
        tgt_len, bsz, embed_dim = x.size()
        assert embed_dim == self.embed_dim
        k = v = None
        if full_cache is not None:
            k, v = _check_cache(full_cache, bsz, self.num_heads, self.head_dim, cache_len + tgt_len, x.dtype)
        else:
            assert cache_len == 0
        b_in = self.in_proj.bias if self.in_proj.bias is not None else self._no_in_bias
        b_out = self.out_proj.bias if self.out_proj.bias is not None else self._no_out_bias
        res = _AttentionFunction.apply(self.num_heads, cache_len, x, k, v, self.in_proj.weight, b_in,
                                       self.out_proj.weight, b_out)
        if full_cache is not None:
            return res[0], (res[1], res[2])
        return res, None

    def create_attn_cache(self, batch_size, seq_len, device="cuda", dtype=torch.float32):
        k = torch.zeros(batch_size * self.num_heads, seq_len, self.head_dim, device=device, dtype=dtype)
        v = torch.zeros(batch_size * self.num_heads, seq_len, self.head_dim, device=device, dtype=dtype)
        return k, v


class TransformerLayer(nn.Module):
    """Reference transformer_models.py:264-285: pre-LN block with a ReLU MLP.  (The reference's plain
    class omits `checkpoint_gradients` and cannot run; here it defaults to False.)"""

    # Two switches for loops that call .backward() / autograd.backward slice by slice, as the reference's does
    # (torch.autograd.grad would see None for the parameters, and post-accumulate-grad hooks may not fire):
    # accumulate_grads_in_place -- the backward of a slice adds its parameter gradients to existing .grad tensors
    # inside the gradient kernels instead of returning them to autograd (same sums, one rounding fewer);
    # defer_weight_grads -- with a cache, the weight gradients of a sequence are taken once, over all its rows, in
    # the backward of the slice at cache_len 0, which the reverse-slice order reaches last; .grad is complete when
    # that backward returns, and every slice of the sequence must run its backward, last slice first.
    accumulate_grads_in_place = False
    defer_weight_grads = False

    def __init__(self, embedding_dim, ffn_embedding_dim, num_attention_heads, device="cpu",
                 checkpoint_gradients=False, activation="relu"):
        super().__init__()
        self.checkpoint_gradients = checkpoint_gradients
        self.activation = activation
        self._grad_options = _GradOptions()
        self.attn_ln = nn.LayerNorm(embedding_dim).to(device)
        self.attn = MultiheadLMAttentionWithCache(embedding_dim, num_attention_heads, device=device)
        self.fc_ln = nn.LayerNorm(embedding_dim).to(device)
        self.fc1 = ColumnParallelLinear(embedding_dim, ffn_embedding_dim, gather_output=False, device=device)
        self.fc2 = RowParallelLinear(ffn_embedding_dim, embedding_dim, input_is_parallel=True, device=device)

    def param_dict(self):
        """The 12 parameter tensors keyed by their state-dict names."""
        return {"attn_ln.weight": self.attn_ln.weight, "attn_ln.bias": self.attn_ln.bias,
                "attn.in_proj.weight": self.attn.in_proj.weight, "attn.in_proj.bias": self.attn.in_proj.bias,
                "attn.out_proj.weight": self.attn.out_proj.weight, "attn.out_proj.bias": self.attn.out_proj.bias,
                "fc_ln.weight": self.fc_ln.weight, "fc_ln.bias": self.fc_ln.bias,
                "fc1.weight": self.fc1.weight, "fc1.bias": self.fc1.bias,
                "fc2.weight": self.fc2.weight, "fc2.bias": self.fc2.bias}

    def forward(self, x, full_cache=None, cache_len=0):
        tgt_len, bsz, embed_dim = x.size()
        assert embed_dim == self.attn.embed_dim
        k = v = None
        if full_cache is not None:
            k, v = _check_cache(full_cache, bsz, self.attn.num_heads, self.attn.head_dim, cache_len + tgt_len, x.dtype)
        else:
            assert cache_len == 0
        p = self.param_dict()
        opts = self._grad_options
        opts.in_place, opts.defer = bool(self.accumulate_grads_in_place), bool(self.defer_weight_grads)
        res = _LayerFunction.apply(self.attn.num_heads, cache_len, self.activation, opts,
                                   x, k, v, *[p[n] for n in core.PARAM_NAMES])
        if full_cache is not None:
            return res[0], (res[1], res[2])
        return res, None


class ModelParallelMultiheadLMAttentionWithCache(MultiheadLMAttentionWithCache):
    """Reference transformer_models.py:288-311 at model-parallel size 1."""

    def __init__(self, embed_dim, num_heads, bias=True, device="cpu"):
        super().__init__(embed_dim, num_heads, bias=bias, device=device)
        self.model_parallel_size = 1
        self.num_total_heads = num_heads


class ModelParallelTransformerLayer(TransformerLayer):
    """Reference transformer_models.py:314-327 at model-parallel size 1 (the class the reference runs)."""

    def __init__(self, embedding_dim, ffn_embedding_dim, num_attention_heads, device="cpu",
                 checkpoint_gradients=False, activation="relu"):
        super().__init__(embedding_dim, ffn_embedding_dim, num_attention_heads, device=device,
                         checkpoint_gradients=checkpoint_gradients, activation=activation)
        self.model_parallel_size = 1


class SingleDeviceTransformer(nn.Module):
    """Reference transformer_models.py:330-342."""

    def __init__(self, transformer_layers):
        super().__init__()
        self.layers = nn.ModuleList(transformer_layers)

    def forward(self, x, attn_caches=None):
        if attn_caches is None:
            attn_caches = [None] * len(self.layers)
        new_attn_caches = []
        for layer, attn_cache in zip(self.layers, attn_caches):
            x, new_attn_cache = layer(x, attn_cache)
            new_attn_caches.append(new_attn_cache)
        return x, new_attn_caches


# ------------------------------------------------------------------------------------------------
# slicers (reference transformer_models.py:368-409)
# ------------------------------------------------------------------------------------------------
def uniform_slice_x(x, n_slices):
    seq_len = x.size(0)
    out, start = [], 0
    for i in range(n_slices):
        n = seq_len // n_slices + int(i < seq_len % n_slices)
        out.append(x[start:start + n])
        start += n
    assert start == seq_len
    return out


def grid_slice_batch_and_sequence(x, batch_slices, seq_slices, requires_grad=False, batch_dim=1, sequence_dim=0):
    """Object ndarray [n_batch_slices, n_seq_slices] of detached contiguous copies."""
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
