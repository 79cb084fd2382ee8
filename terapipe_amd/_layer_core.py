"""Functional core of one GPT layer over one sequence slice: the kernel sequence for forward and
backward, shared by the autograd wrappers in transformer_models.py and by the sliced runner in
terapipe.py.  Follows TransformerLayer.forward (transformer_models.py:273-285 of the reference) and
MultiheadLMAttentionWithCache.forward (:214-255); every arithmetic step is a call into
libterapipe_hip.so through terapipe_amd.ops.
"""
import torch

from . import ops
from ._lib import (TP_EPI_BIAS_GELU, TP_EPI_BIAS_RELU, TP_EPI_BIAS_RESIDUAL, TP_EPI_GELU_GRAD, TP_EPI_QKV_SCATTER,
                   TP_EPI_RELU_GRAD, TP_GEMM_NN, TP_GEMM_NT)

# order of the small (vector) parameters inside one layer's fp32 gradient accumulator
SMALL_PARAMS = ("attn_ln.weight", "attn_ln.bias", "attn.in_proj.bias", "attn.out_proj.bias",
                "fc_ln.weight", "fc_ln.bias", "fc1.bias", "fc2.bias")
BIG_PARAMS = ("attn.in_proj.weight", "attn.out_proj.weight", "fc1.weight", "fc2.weight")
PARAM_NAMES = ("attn_ln.weight", "attn_ln.bias", "attn.in_proj.weight", "attn.in_proj.bias",
               "attn.out_proj.weight", "attn.out_proj.bias", "fc_ln.weight", "fc_ln.bias",
               "fc1.weight", "fc1.bias", "fc2.weight", "fc2.bias")


def small_param_sizes(E, F):
    return {"attn_ln.weight": E, "attn_ln.bias": E, "attn.in_proj.bias": 3 * E, "attn.out_proj.bias": E,
            "fc_ln.weight": E, "fc_ln.bias": E, "fc1.bias": F, "fc2.bias": E}


def small_acc_views(buf, E, F):
    """Splits a flat fp32 buffer of small_acc_numel(E, F) elements into per-parameter views."""
    views, off = {}, 0
    for name in SMALL_PARAMS:
        n = small_param_sizes(E, F)[name]
        views[name] = buf[off:off + n]
        off += n
    return views


def small_acc_numel(E, F):
    return sum(small_param_sizes(E, F).values())


class SliceState:
    """What one layer keeps from the forward of one slice for its backward."""
    __slots__ = ("x", "mean1", "rstd1", "xn", "q", "o", "lse", "h", "mean2", "rstd2", "hn", "a", "z",
                 "k_cache", "v_cache", "cache_len", "T", "B", "q_bh_rows", "stat_bh_rows")


class Bufs:
    """Optional preallocated outputs for one layer-slice call (views into the runner's per-layer
    buffers).  Any attribute left at None is allocated by the call.  q_bh_rows / stat_bh_rows: q and
    lse / delta are views, starting at the slice's position, into position-indexed buffers with that many
    rows per (batch, head) -- 0 means compact [B*H, T, ...] tensors.  x_pending: the layer input is still the
    partial sums of the previous layer's k-split fc2 GEMM (ops.PendingReduce) and the first LayerNorm
    finishes it; defer_out: leave this layer's fc2 output in that state, returned in out_pending.
    sync: called (no arguments) at the one point of the layer where a slice depends on other slices: in forward
    after the in_proj GEMM has been launched and before the attention kernel (which reads the K/V rows the
    earlier slices' in_proj GEMMs write), in backward between the dQ kernel (which leaves this slice's delta)
    and the one-pass dK/dV kernel (which reads dO and delta of every later slice).  A runner that spreads
    slices over streams waits for / records its events there."""
    __slots__ = ("xn", "mean1", "rstd1", "q", "o", "lse", "h", "mean2", "rstd2", "hn", "a", "z", "out",
                 "dz1", "dhn", "dh", "d_o", "dqkv", "dxn", "dx", "delta", "q_bh_rows", "stat_bh_rows",
                 "x_pending", "defer_out", "out_pending", "sync")

    def __init__(self, **kw):
        for n in self.__slots__:
            setattr(self, n, kw.get(n))
        self.q_bh_rows = self.q_bh_rows or 0
        self.stat_bh_rows = self.stat_bh_rows or 0


_NOBUF = Bufs()


def _buf(t, shape, dtype, device):
    return torch.empty(shape, dtype=dtype, device=device) if t is None else t


def attention_fwd(w, xn2d, T, B, heads, k_cache, v_cache, cache_len, buf=_NOBUF):
    """in_proj GEMM with the q/k/v split, q scaling and cache assignment fused into its epilogue, then
    the prefix-cached attention kernel.  Returns q [B*H, T, Dh], o [T, B, E], lse."""
    E = xn2d.shape[1]
    Dh = E // heads
    M = T * B
    q = _buf(buf.q, (B * heads, T, Dh), xn2d.dtype, xn2d.device)
    scale = float(Dh) ** -0.5
    ops.gemm(TP_GEMM_NT, xn2d, w["attn.in_proj.weight"], M, 3 * E, E, epilogue=TP_EPI_QKV_SCATTER,
             bias=w["attn.in_proj.bias"],
             qkv=dict(q=q, k_cache=k_cache, v_cache=v_cache, batch=B, heads=heads, head_dim=Dh,
                      cache_len=cache_len, cache_rows=k_cache.shape[1], q_scale=scale, q_bh_rows=buf.q_bh_rows))
    if buf.sync is not None:
        buf.sync()
    o, lse = ops.attn_prefix_fwd(q, k_cache, v_cache, B, heads, Dh, T, cache_len, scale, out=buf.o, lse=buf.lse,
                                 q_bh_rows=buf.q_bh_rows, stat_bh_rows=buf.stat_bh_rows)
    return q, o, lse


def layer_fwd(w, x, heads, k_cache, v_cache, cache_len, activation="relu", need_state=True, buf=_NOBUF):
    """x [T, B, E] contiguous.  Writes rows [cache_len, cache_len+T) of the caches.  Returns (out, state)."""
    T, B, E = x.shape
    M = T * B
    F = w["fc1.weight"].shape[0]
    dt, dev = x.dtype, x.device
    x2d = x.view(M, E)
    xn, mean1, rstd1 = ops.layernorm_fwd(buf.x_pending if buf.x_pending is not None else x2d, w["attn_ln.weight"],
                                         w["attn_ln.bias"], out=buf.xn, mean=buf.mean1, rstd=buf.rstd1)
    q, o, lse = attention_fwd(w, xn, T, B, heads, k_cache, v_cache, cache_len, buf)
    o2d = o.view(M, E)
    h = _buf(buf.h, (M, E), dt, dev)
    # a k-split out_proj leaves its partial sums to the LayerNorm that follows directly (which then writes h)
    h_in = ops.gemm(TP_GEMM_NT, o2d, w["attn.out_proj.weight"], M, E, E, C=h, epilogue=TP_EPI_BIAS_RESIDUAL,
                    bias=w["attn.out_proj.bias"], residual=x2d, defer_reduce=True)
    hn, mean2, rstd2 = ops.layernorm_fwd(h_in, w["fc_ln.weight"], w["fc_ln.bias"], out=buf.hn, mean=buf.mean2,
                                         rstd=buf.rstd2)
    a = _buf(buf.a, (M, F), dt, dev)
    z = None
    if activation == "relu":
        ops.gemm(TP_GEMM_NT, hn, w["fc1.weight"], M, F, E, C=a, epilogue=TP_EPI_BIAS_RELU, bias=w["fc1.bias"])
    elif activation == "gelu":
        z = _buf(buf.z, (M, F), dt, dev)
        ops.gemm(TP_GEMM_NT, hn, w["fc1.weight"], M, F, E, C=a, epilogue=TP_EPI_BIAS_GELU, bias=w["fc1.bias"],
                 aux_out=z)
    else:
        raise ValueError("activation must be 'relu' or 'gelu'")
    out = _buf(buf.out, (M, E), dt, dev)
    res = ops.gemm(TP_GEMM_NT, a, w["fc2.weight"], M, E, F, C=out, epilogue=TP_EPI_BIAS_RESIDUAL,
                   bias=w["fc2.bias"], residual=h, defer_reduce=bool(buf.defer_out))
    if buf.defer_out:
        buf.out_pending = res if isinstance(res, ops.PendingReduce) else None
    st = None
    if need_state:
        st = SliceState()
        st.x, st.mean1, st.rstd1, st.xn = x2d, mean1, rstd1, xn
        st.q, st.o, st.lse = q, o2d, lse
        st.h, st.mean2, st.rstd2, st.hn = h, mean2, rstd2, hn
        st.a, st.z = a, z
        st.k_cache, st.v_cache, st.cache_len, st.T, st.B = k_cache, v_cache, cache_len, T, B
        st.q_bh_rows, st.stat_bh_rows = buf.q_bh_rows, buf.stat_bh_rows
    return out.view(T, B, E), st


def layer_bwd(w, st, dout, heads, gk, gv, accumulate_prefix, has_incoming, zero_slice_rows, activation="relu",
              buf=_NOBUF, suffix=None):
    """Backward of layer_fwd for one slice: the data gradients.

    dout [T, B, E]; gk / gv gradient caches (see tp_attn_desc).  The parameter gradients are the caller's: it
    keeps the intermediate gradients this call leaves in `buf` (dz1, dhn, dh, dqkv, dxn; dout is fc2's) and
    reduces them against the saved inputs -- per slice (the layer-level surface) or over all slices of a step at
    once (the runner): four TN products and eight column reductions (ops.gemm_grouped, ops.vec_param_grads).
    suffix: None, or dict(q_all, d_o_all, lse_all, delta_all, q_end) of position-indexed buffers that hold
    every slice processed so far (buf.d_o and buf.delta are then views of them at this slice): dK/dV of
    the slice's keys are computed in one pass over all later query positions and gk / gv are not used.
    With suffix["fused"] (needs o_all and own_end) dQ and that pass go out as one launch.
    Returns dx [T, B, E].
    """
    T, B = st.T, st.B
    M = T * B
    E = st.x.shape[1]
    F = st.a.shape[1]
    Dh = E // heads
    dt, dev = dout.dtype, dout.device
    dout2d = dout.reshape(M, E)
    # MLP
    dz1 = _buf(buf.dz1, (M, F), dt, dev)
    if activation == "relu":
        ops.gemm(TP_GEMM_NN, dout2d, w["fc2.weight"], M, F, E, C=dz1, epilogue=TP_EPI_RELU_GRAD, aux=st.a)
    else:
        ops.gemm(TP_GEMM_NN, dout2d, w["fc2.weight"], M, F, E, C=dz1, epilogue=TP_EPI_GELU_GRAD, aux=st.z)
    dhn = _buf(buf.dhn, (M, E), dt, dev)
    # a k-split data-gradient GEMM leaves its partial sums to the LayerNorm backward that follows directly
    dhn_in = ops.gemm(TP_GEMM_NN, dz1, w["fc1.weight"], M, E, F, C=dhn, defer_reduce=True)
    dh = ops.layernorm_bwd(dhn_in, st.h, st.mean2, st.rstd2, w["fc_ln.weight"], dout2d, None, None, None, None,
                           out=buf.dh)
    # attention
    d_o = _buf(buf.d_o, (M, E), dt, dev)
    ops.gemm(TP_GEMM_NN, dh, w["attn.out_proj.weight"], M, E, E, C=d_o)
    dqkv = _buf(buf.dqkv, (M, 3 * E), dt, dev)
    if suffix is None:
        ops.attn_prefix_bwd(st.q, st.k_cache, st.v_cache, st.o, st.lse, d_o, dqkv, gk, gv, B, heads, Dh, T,
                            st.cache_len, float(Dh) ** -0.5, accumulate_prefix, has_incoming, zero_slice_rows,
                            delta=buf.delta,
                            q_bh_rows=st.q_bh_rows, stat_bh_rows=st.stat_bh_rows)
    elif suffix.get("fused"):
        # dQ of the slice and dK / dV of its keys over all later positions as one launch.  The dK/dV half takes delta
        # of the positions up to own_end itself, so what it needs of the later slices is their dO (and, past own_end,
        # their delta): the slice waits for the next slice's event and records its own BEFORE the launch.  (An event
        # recorded there does not cover this launch's delta: the caller may only mix fused and two-launch slices
        # on ONE stream, see terapipe.fused_backward_slices.)
        if buf.sync is not None:
            buf.sync()
        ops.attn_bwd_fused(st.q, st.k_cache, st.v_cache, st.o, st.lse, d_o, dqkv, B, heads, Dh, T, st.cache_len,
                           float(Dh) ** -0.5, buf.delta, suffix["q_all"], suffix["d_o_all"], suffix["lse_all"],
                           suffix["delta_all"], suffix["o_all"], suffix["q_end"], suffix["own_end"],
                           q_bh_rows=st.q_bh_rows, stat_bh_rows=st.stat_bh_rows)
    else:
        ops.attn_prefix_bwd(st.q, st.k_cache, st.v_cache, st.o, st.lse, d_o, dqkv, None, None, B, heads, Dh, T,
                            st.cache_len, float(Dh) ** -0.5, False, False, False, delta=buf.delta,
                            q_bh_rows=st.q_bh_rows, stat_bh_rows=st.stat_bh_rows, dq_only=True)
        if buf.sync is not None:
            buf.sync()
        ops.attn_suffix_dkdv(st.k_cache, st.v_cache, suffix["q_all"], suffix["d_o_all"], suffix["lse_all"],
                             suffix["delta_all"], dqkv, B, heads, Dh, st.cache_len, T, suffix["q_end"])
    dxn = _buf(buf.dxn, (M, E), dt, dev)
    dxn_in = ops.gemm(TP_GEMM_NN, dqkv, w["attn.in_proj.weight"], M, E, 3 * E, C=dxn, defer_reduce=True)
    dx = ops.layernorm_bwd(dxn_in, st.x, st.mean1, st.rstd1, w["attn_ln.weight"], dh, None, None, None, None,
                           out=buf.dx)
    return dx.view(T, B, E)
