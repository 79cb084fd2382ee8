"""Thin torch-tensor wrappers over the C ABI (include/terapipe_hip.h).

PyTorch owns all device memory and the stream; these functions only pass ``data_ptr()``s, shapes and
``torch.cuda.current_stream()`` to the library.  Nothing here computes on the host and nothing falls
back to PyTorch kernels: a missing library or a non-zero status raises.
"""
import ctypes

import torch

from . import _lib
from ._lib import (AttnDesc, GemmDesc, TP_BF16, TP_F16, TP_F32, TP_GEMM_NN, TP_GEMM_NT, TP_GEMM_TN,
                   TP_EPI_ACCUMULATE, TP_EPI_BIAS, TP_EPI_BIAS_GELU, TP_EPI_BIAS_RELU, TP_EPI_BIAS_RESIDUAL,
                   TP_EPI_GELU_GRAD, TP_EPI_QKV_SCATTER, TP_EPI_RELU_GRAD, TP_EPI_STORE)

_DTYPES = {torch.float32: TP_F32, torch.float16: TP_F16, torch.bfloat16: TP_BF16}


def tp_dtype(dtype):
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise TypeError("unsupported dtype %s (float32, float16, bfloat16)" % dtype)


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _p(t):
    return None if t is None else t.data_ptr()


def _require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise _lib.TeraPipeHipError("terapipe_amd kernels need CUDA/HIP tensors; there is no CPU path")


class CallRecorder:
    """Records every library call made while active as (tag, meta, replay) where replay(stream=None) issues
    the same call again with the same descriptor and buffers, on the given stream handle or else on the
    then-current stream.  bench.py replays all calls of one kind back to back inside a HIP graph to time that
    kind of kernel without host gaps.  With ``program`` set to a list, every call is also appended to it as
    (replay, stream handle it was issued on): the runner interleaves its stream waits and event records in the
    same list and re-issues the whole step from it without rebuilding a single descriptor."""
    active = None

    def __init__(self, program=None):
        self.calls = []
        self.program = program

    def __enter__(self):
        CallRecorder.active = self
        return self

    def __exit__(self, *exc):
        CallRecorder.active = None

    def by_tag(self, tag):
        return [c for c in self.calls if c[0] == tag]


def _record(tag, meta, replay):
    rec = CallRecorder.active
    if rec is not None:
        rec.calls.append((tag, meta, replay))
        if rec.program is not None:
            rec.program.append((replay, _stream()))


def _on(stream):
    return _stream() if stream is None else stream


# (op, M, N, K) -> (tile configuration, k splits): overrides the library's plan for that shape.  A tuning hook:
# terapipe_amd.tune_gemm's in-step search fills it to time whole steps with one shape's plan changed.
GEMM_PLAN_OVERRIDE = {}


class Workspace:
    """A grow-only scratch tensor per device and stream (torch-owned), handed to calls that need
    workspace: kernels of different streams may run at the same time and must not share partial sums.
    A buffer that is outgrown is kept for the life of the process, never returned to torch's allocator:
    recorded launches and captured HIP graphs hold its raw address and may run again at any time.  A new
    buffer is at least half as large again as the one it replaces, so that the outgrown ones of a stream
    add up to no more than twice its current buffer however the requests creep up."""
    _bufs = {}
    _superseded = []

    @classmethod
    def get(cls, nbytes, device, stream=None):
        """The buffer of `stream` (a raw stream handle; default: the current stream), grown to nbytes if needed."""
        if stream is None:
            stream = torch.cuda.current_stream(device).cuda_stream
        key = (device.type, device.index, stream)
        buf = cls._bufs.get(key)
        if buf is None or buf.numel() < nbytes:
            size = max(int(nbytes), 1 << 20)
            if buf is not None:
                cls._superseded.append(buf)
                size = max(size, buf.numel() + buf.numel() // 2)
            buf = torch.empty(size, dtype=torch.uint8, device=device)
            cls._bufs[key] = buf
        return buf

    @classmethod
    def size(cls, device, stream):
        buf = cls._bufs.get((device.type, device.index, stream))
        return 0 if buf is None else buf.numel()


class PendingReduce:
    """What gemm(..., defer_reduce=True) returns when the plan splits k: the fp32 partial sums are in `ws`
    and the tensor `out` is NOT written yet.  layernorm_fwd / layernorm_bwd accept it in place of their input
    tensor and then also produce `out` (sum of the partials + bias + residual, rounded to out's dtype).  It
    must be consumed before the next split-k GEMM of the same stream reuses the workspace."""
    __slots__ = ("ws", "nsplit", "bias", "residual", "out")

    def __init__(self, ws, nsplit, bias, residual, out):
        self.ws, self.nsplit, self.bias, self.residual, self.out = ws, nsplit, bias, residual, out


def layernorm_fwd(x2d, gamma, beta, eps=1e-5, out=None, mean=None, rstd=None):
    """x2d: the input rows, or a PendingReduce (then x2d.out is written as well)."""
    pend = x2d if isinstance(x2d, PendingReduce) else None
    if pend is not None:
        x2d = pend.out
    _require_cuda(x2d, gamma, beta)
    M, E = x2d.shape
    y = torch.empty_like(x2d) if out is None else out
    mean = torch.empty(M, dtype=torch.float32, device=x2d.device) if mean is None else mean
    rstd = torch.empty(M, dtype=torch.float32, device=x2d.device) if rstd is None else rstd
    lib = _lib.load()
    if pend is not None:
        a = (_p(pend.ws), pend.nsplit, _p(pend.bias), _p(pend.residual), _p(x2d), _p(gamma), _p(beta), _p(y), _p(mean),
             _p(rstd), M, E, eps, tp_dtype(x2d.dtype))
        _lib.check(lib.tp_layernorm_fwd_partials(*a, _stream()), "tp_layernorm_fwd_partials")
        _record("layernorm_fwd", (M, E), lambda s=None, keep=pend: lib.tp_layernorm_fwd_partials(*a, _on(s)))
        return y, mean, rstd
    _lib.check(lib.tp_layernorm_fwd(_p(x2d), _p(gamma), _p(beta), _p(y), _p(mean), _p(rstd), M, E, eps,
                                    tp_dtype(x2d.dtype), _stream()), "tp_layernorm_fwd")
    if CallRecorder.active is not None:
        a = (_p(x2d), _p(gamma), _p(beta), _p(y), _p(mean), _p(rstd), M, E, eps, tp_dtype(x2d.dtype))
        _record("layernorm_fwd", (M, E), lambda s=None: lib.tp_layernorm_fwd(*a, _on(s)))
    return y, mean, rstd


def layernorm_bwd(dy, x2d, mean, rstd, gamma, dres, dgamma_acc, dbeta_acc, colsum_dres_acc=None,
                  colsum_dx_acc=None, out=None):
    """dgamma_acc / dbeta_acc may be None: then only dx is computed (the parameter gradients are left
    to ln_param_grads over all rows).  dy: the gradient rows, or a PendingReduce (then dy.out is written)."""
    pend = dy if isinstance(dy, PendingReduce) else None
    if pend is not None:
        dy = pend.out
    _require_cuda(dy, x2d, gamma)
    M, E = x2d.shape
    dx = torch.empty_like(x2d) if out is None else out
    lib = _lib.load()
    if pend is not None:
        a = (_p(pend.ws), pend.nsplit, _p(dy), _p(x2d), _p(mean), _p(rstd), _p(gamma), _p(dres), _p(dx), _p(dgamma_acc),
             _p(dbeta_acc), _p(colsum_dres_acc), _p(colsum_dx_acc), M, E, tp_dtype(x2d.dtype))
        _lib.check(lib.tp_layernorm_bwd_partials(*a, _stream()), "tp_layernorm_bwd_partials")
        _record("layernorm_bwd", (M, E), lambda s=None, keep=pend: lib.tp_layernorm_bwd_partials(*a, _on(s)))
        return dx
    _lib.check(lib.tp_layernorm_bwd(_p(dy), _p(x2d), _p(mean), _p(rstd), _p(gamma), _p(dres), _p(dx),
                                    _p(dgamma_acc), _p(dbeta_acc), _p(colsum_dres_acc), _p(colsum_dx_acc),
                                    M, E, tp_dtype(x2d.dtype), _stream()), "tp_layernorm_bwd")
    if CallRecorder.active is not None:
        a = (_p(dy), _p(x2d), _p(mean), _p(rstd), _p(gamma), _p(dres), _p(dx), _p(dgamma_acc), _p(dbeta_acc),
             _p(colsum_dres_acc), _p(colsum_dx_acc), M, E, tp_dtype(x2d.dtype))
        _record("layernorm_bwd", (M, E), lambda s=None: lib.tp_layernorm_bwd(*a, _on(s)))
    return dx


def gemm(op, A, B, M, N, K, C=None, epilogue=TP_EPI_STORE, bias=None, residual=None, aux=None, aux_out=None,
         colsum_acc=None, qkv=None, tile_cfg=None, ksplit=None, defer_reduce=False, desc_sink=None):
    """Runs one GEMM.  A, B, C, residual, aux are 2-D row-major tensors (stride(1) == 1).
    qkv = dict(q, k_cache, v_cache, batch, heads, head_dim, cache_len, cache_rows, q_scale).
    tile_cfg / ksplit force a tile configuration / k-split count (tuning and tests); default automatic.
    defer_reduce (STORE / BIAS_RESIDUAL epilogues): if the plan splits k, C is left unwritten and a
    PendingReduce is returned for the LayerNorm call that consumes C; otherwise C as usual.
    desc_sink: a list that receives the call's descriptor (the one a recorded replay re-issues), for callers
    that re-point C before a replay."""
    _require_cuda(A, B, C)
    d = GemmDesc()
    d.op, d.dtype, d.epilogue = op, tp_dtype(A.dtype), epilogue
    d.M, d.N, d.K = M, N, K
    d.A, d.lda = A.data_ptr(), A.stride(0)
    d.B, d.ldb = B.data_ptr(), B.stride(0)
    if C is not None:
        d.C, d.ldc = C.data_ptr(), C.stride(0)
    d.bias = _p(bias)
    if residual is not None:
        d.residual, d.ldr = residual.data_ptr(), residual.stride(0)
    if aux is not None:
        d.aux, d.ldaux = aux.data_ptr(), aux.stride(0)
    if aux_out is not None:
        d.aux_out, d.ldauxo = aux_out.data_ptr(), aux_out.stride(0)
    d.colsum_acc = _p(colsum_acc)
    if qkv is not None:
        d.q, d.k_cache, d.v_cache = qkv["q"].data_ptr(), qkv["k_cache"].data_ptr(), qkv["v_cache"].data_ptr()
        d.batch, d.heads, d.head_dim = qkv["batch"], qkv["heads"], qkv["head_dim"]
        d.cache_len, d.cache_rows, d.q_scale = qkv["cache_len"], qkv["cache_rows"], qkv["q_scale"]
        d.q_bh_rows = qkv.get("q_bh_rows", 0)
    if tile_cfg is None and ksplit is None and GEMM_PLAN_OVERRIDE:
        tile_cfg, ksplit = GEMM_PLAN_OVERRIDE.get((op, M, N, K), (None, None))
    if tile_cfg is not None or ksplit is not None:
        d.reserved = ((tile_cfg + 1) if tile_cfg is not None else 0) | ((ksplit or 0) << 8)
    if desc_sink is not None:
        desc_sink.append(d)
    lib = _lib.load()
    nsplit = 1
    if defer_reduce:
        nsplit = lib.tp_gemm_splits(ctypes.byref(d))
        if nsplit > 1:
            d.defer_reduce = 1
    need = lib.tp_gemm_workspace_bytes(ctypes.byref(d))
    ws = Workspace.get(need, A.device) if need else None
    _lib.check(lib.tp_gemm(ctypes.byref(d), _p(ws), ws.numel() if ws is not None else 0, _stream()), "tp_gemm")
    if CallRecorder.active is not None:
        # the closure holds the workspace tensor, not just its address: the memory stays allocated for as
        # long as the recorded call can be re-issued
        wsn = ws.numel() if ws is not None else 0
        _record("gemm", (op, M, N, K), lambda s=None, ws=ws: lib.tp_gemm(ctypes.byref(d), _p(ws), wsn, _on(s)))
    if nsplit > 1:
        return PendingReduce(ws, nsplit, bias, residual, C)
    return C


def gemm_grouped(items, desc_sinks=None):
    """Plain products (epilogue STORE or ACCUMULATE) as one library call: items is a list of
    (op, A, B, M, N, K, C, epilogue).  The library runs the group as one launch when its members allow it and
    one after the other otherwise; the result is that of ``gemm`` on every item in order.
    desc_sinks: per item a list (or None) that receives the item's descriptor, as ``gemm``'s desc_sink."""
    n = len(items)
    descs = (GemmDesc * n)()
    lib = _lib.load()
    need = 0
    for i, (op, A, B, M, N, K, C, epilogue) in enumerate(items):
        _require_cuda(A, B, C)
        d = descs[i]                        # a view into the array
        d.op, d.dtype, d.epilogue = op, tp_dtype(A.dtype), epilogue
        d.M, d.N, d.K = M, N, K
        d.A, d.lda = A.data_ptr(), A.stride(0)
        d.B, d.ldb = B.data_ptr(), B.stride(0)
        d.C, d.ldc = C.data_ptr(), C.stride(0)
        if GEMM_PLAN_OVERRIDE and (op, M, N, K) in GEMM_PLAN_OVERRIDE:
            tile_cfg, ksplit = GEMM_PLAN_OVERRIDE[(op, M, N, K)]
            d.reserved = ((tile_cfg + 1) if tile_cfg is not None else 0) | ((ksplit or 0) << 8)
        if desc_sinks is not None and desc_sinks[i] is not None:
            desc_sinks[i].append(d)
        need = max(need, lib.tp_gemm_workspace_bytes(ctypes.byref(d)))
    ws = Workspace.get(need, items[0][1].device) if need else None
    wsp, wsn = _p(ws), (ws.numel() if ws is not None else 0)
    meta = tuple((op, M, N, K) for (op, _, _, M, N, K, _, _) in items)
    _lib.check(lib.tp_gemm_grouped(descs, n, wsp, wsn, _stream()), "tp_gemm_grouped")
    _record("gemm", meta, lambda s=None, ws=ws: lib.tp_gemm_grouped(descs, n, _p(ws), wsn, _on(s)))


def _attn_desc(q, k_cache, v_cache, o, lse, batch, heads, head_dim, T, cache_len, q_scale, q_bh_rows=0,
               stat_bh_rows=0):
    """q_bh_rows / stat_bh_rows: rows per (batch, head) block of q / of lse and delta when these are views
    into position-indexed buffers that hold every slice (0 = compact [B*H, T, ...])."""
    d = AttnDesc()
    d.q_bh_rows, d.stat_bh_rows = q_bh_rows, stat_bh_rows
    d.dtype = tp_dtype(q.dtype)
    d.batch, d.heads, d.head_dim, d.T, d.cache_len = batch, heads, head_dim, T, cache_len
    d.cache_rows = k_cache.shape[1]
    d.q, d.k_cache, d.v_cache, d.o, d.lse = q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), o.data_ptr(), lse.data_ptr()
    d.q_scale = q_scale
    return d


def attn_prefix_fwd(q, k_cache, v_cache, batch, heads, head_dim, T, cache_len, q_scale, out=None, lse=None,
                    nsplit=None, q_bh_rows=0, stat_bh_rows=0, variant=0):
    """q [B*H, T, Dh] (pre-scaled); caches [B*H, L, Dh] with rows [0, cache_len+T) valid.
    Returns o [T, B, H*Dh] and lse [B*H, T]."""
    _require_cuda(q, k_cache, v_cache)
    o = torch.empty(T, batch, heads * head_dim, dtype=q.dtype, device=q.device) if out is None else out
    if lse is None:
        lse = torch.empty(batch * heads, T, dtype=torch.float32, device=q.device)
    d = _attn_desc(q, k_cache, v_cache, o, lse, batch, heads, head_dim, T, cache_len, q_scale, q_bh_rows, stat_bh_rows)
    if nsplit:
        d.reserved = int(nsplit)
    if variant:
        d.reserved2 = int(variant)      # tuning / tests: see tp_attn_desc.reserved2
    lib = _lib.load()
    need = lib.tp_attn_fwd_workspace_bytes(ctypes.byref(d))
    ws = Workspace.get(need, q.device) if need else None
    _lib.check(lib.tp_attn_prefix_fwd(ctypes.byref(d), _p(ws), ws.numel() if ws is not None else 0, _stream()),
               "tp_attn_prefix_fwd")
    if CallRecorder.active is not None:
        wsn = ws.numel() if ws is not None else 0
        _record("attn_fwd", (batch, heads, head_dim, T, cache_len),
                lambda s=None, ws=ws: lib.tp_attn_prefix_fwd(ctypes.byref(d), _p(ws), wsn, _on(s)))
    return o, lse


def attn_prefix_bwd(q, k_cache, v_cache, o, lse, d_o, dqkv, dk_cache, dv_cache, batch, heads, head_dim, T,
                    cache_len, q_scale, accumulate_prefix, has_incoming, zero_slice_rows, colsum_dqkv_acc=None,
                    delta=None, q_bh_rows=0, stat_bh_rows=0, dq_only=False):
    """Writes dqkv [T*B, 3*H*Dh]; updates rows [0, cache_len) of the gradient caches.  dq_only: delta and
    the q part of dqkv only (the k and v parts are then attn_suffix_dkdv's; no gradient cache is touched)."""
    _require_cuda(q, k_cache, v_cache, d_o, dqkv)
    if delta is None:
        delta = torch.empty(batch * heads, T, dtype=torch.float32, device=q.device)
    d = _attn_desc(q, k_cache, v_cache, o, lse, batch, heads, head_dim, T, cache_len, q_scale, q_bh_rows, stat_bh_rows)
    d.dq_only = int(dq_only)
    d.d_o, d.delta, d.dqkv = d_o.data_ptr(), delta.data_ptr(), dqkv.data_ptr()
    d.dk_cache, d.dv_cache = _p(dk_cache), _p(dv_cache)
    d.grad_cache_dtype = tp_dtype(dk_cache.dtype) if dk_cache is not None else d.dtype
    d.accumulate_prefix, d.has_incoming, d.zero_slice_rows = int(accumulate_prefix), int(has_incoming), int(zero_slice_rows)
    d.colsum_dqkv_acc = _p(colsum_dqkv_acc)
    lib = _lib.load()
    _lib.check(lib.tp_attn_prefix_bwd(ctypes.byref(d), None, 0, _stream()), "tp_attn_prefix_bwd")
    _record("attn_bwd", (batch, heads, head_dim, T, cache_len),
            lambda s=None: lib.tp_attn_prefix_bwd(ctypes.byref(d), None, 0, _on(s)))
    return dqkv


def attn_suffix_dkdv(k_cache, v_cache, q_all, d_o_all, lse_all, delta_all, dqkv, batch, heads, head_dim,
                     key_begin, key_count, q_end):
    """dK / dV of the keys [key_begin, key_begin + key_count) against every query position in
    [key_begin, q_end), written into the k and v parts of dqkv [key_count * B, 3 * H * Dh].
    q_all [B*H, Lq, Dh], lse_all / delta_all [B*H, Ls], d_o_all [>= q_end, B, H*Dh]: all indexed by position."""
    _require_cuda(k_cache, v_cache, q_all, d_o_all, dqkv)
    d = _lib.AttnSuffixDesc()
    d.dtype = tp_dtype(q_all.dtype)
    d.batch, d.heads, d.head_dim = batch, heads, head_dim
    d.key_begin, d.key_count, d.q_end = key_begin, key_count, q_end
    d.cache_rows, d.q_bh_rows, d.stat_bh_rows = k_cache.shape[1], q_all.shape[1], lse_all.shape[1]
    d.k_cache, d.v_cache = k_cache.data_ptr(), v_cache.data_ptr()
    d.q_all, d.d_o_all = q_all.data_ptr(), d_o_all.data_ptr()
    d.lse_all, d.delta_all, d.dqkv = lse_all.data_ptr(), delta_all.data_ptr(), dqkv.data_ptr()
    lib = _lib.load()
    _lib.check(lib.tp_attn_suffix_dkdv(ctypes.byref(d), _stream()), "tp_attn_suffix_dkdv")
    _record("attn_bwd_dkdv", (batch, heads, head_dim, key_count, key_begin),
            lambda s=None: lib.tp_attn_suffix_dkdv(ctypes.byref(d), _on(s)))
    return dqkv


# The fused backward launch takes the delta of a window of positions itself (its own slice's and those of the slices
# whose launches may still be running); the library accepts up to 4096.  Every dK/dV workgroup recomputes the window's
# delta, which pays while the window is short: measured with three slice streams, 32-token slices (window 96) gain
# 1 % of the step and 36 % on the attention backward alone, slices of 128 tokens and more (windows from 384) lose
# 0.3-2.5 % of the step.  The runner fuses up to this window.
FUSED_BWD_WINDOW = 128


def attn_bwd_fused(q, k_cache, v_cache, o, lse, d_o, dqkv, batch, heads, head_dim, T, cache_len, q_scale, delta,
                   q_all, d_o_all, lse_all, delta_all, o_all, q_end, own_delta_end=None, q_bh_rows=0, stat_bh_rows=0):
    """attn_prefix_bwd(dq_only=True) and attn_suffix_dkdv of the same slice as one launch (fp16 / bf16): writes
    delta and all three parts of dqkv [T*B, 3*H*Dh].  Arguments as in the two calls; the slice is the positions
    [cache_len, cache_len + T) and queries up to q_end take part in its dK / dV.  o_all [>= q_end, B, H*Dh] is the
    attention output by position; delta of the positions [cache_len, own_delta_end) is taken inside the launch
    (default: the slice's own), delta_all is read only from own_delta_end on."""
    _require_cuda(q, k_cache, v_cache, d_o, dqkv, q_all, d_o_all, o_all)
    d = _attn_desc(q, k_cache, v_cache, o, lse, batch, heads, head_dim, T, cache_len, q_scale, q_bh_rows, stat_bh_rows)
    d.dq_only = 1
    d.d_o, d.delta, d.dqkv = d_o.data_ptr(), delta.data_ptr(), dqkv.data_ptr()
    d.grad_cache_dtype = d.dtype
    sd = _lib.AttnSuffixDesc()
    sd.dtype = d.dtype
    sd.batch, sd.heads, sd.head_dim = batch, heads, head_dim
    sd.key_begin, sd.key_count, sd.q_end = cache_len, T, q_end
    sd.cache_rows, sd.q_bh_rows, sd.stat_bh_rows = k_cache.shape[1], q_all.shape[1], lse_all.shape[1]
    sd.k_cache, sd.v_cache = k_cache.data_ptr(), v_cache.data_ptr()
    sd.q_all, sd.d_o_all = q_all.data_ptr(), d_o_all.data_ptr()
    sd.lse_all, sd.delta_all, sd.dqkv = lse_all.data_ptr(), delta_all.data_ptr(), dqkv.data_ptr()
    own_end = cache_len + T if own_delta_end is None else int(own_delta_end)
    o_ptr = o_all.data_ptr()
    lib = _lib.load()
    _lib.check(lib.tp_attn_bwd_fused(ctypes.byref(d), ctypes.byref(sd), o_ptr, own_end, _stream()), "tp_attn_bwd_fused")
    _record("attn_bwd", (batch, heads, head_dim, T, cache_len),
            lambda s=None: lib.tp_attn_bwd_fused(ctypes.byref(d), ctypes.byref(sd), o_ptr, own_end, _on(s)))
    return dqkv


def ln_param_grads(dy, x2d, mean, rstd, dgamma_acc, dbeta_acc):
    """dgamma_acc[E] += sum_m dy * xhat, dbeta_acc[E] += sum_m dy over all M rows (fp32 accumulators)."""
    _require_cuda(dy, x2d, dgamma_acc, dbeta_acc)
    M, E = x2d.shape
    lib = _lib.load()
    _lib.check(lib.tp_ln_param_grads(_p(dy), _p(x2d), _p(mean), _p(rstd), _p(dgamma_acc), _p(dbeta_acc), M, E,
                                     tp_dtype(x2d.dtype), _stream()), "tp_ln_param_grads")
    if CallRecorder.active is not None:
        a = (_p(dy), _p(x2d), _p(mean), _p(rstd), _p(dgamma_acc), _p(dbeta_acc), M, E, tp_dtype(x2d.dtype))
        _record("ln_param_grads", (M, E), lambda s=None: lib.tp_ln_param_grads(*a, _on(s)))


def vec_param_grads(problems):
    """Up to 8 reductions over the rows of a step in one launch.  problems: (dy, acc) for a column sum
    (acc[N] += sum_m dy[m]) or (dy, x, mean, rstd, dgamma_acc, dbeta_acc) for a LayerNorm pair; every dy / x is a
    2-D row-major tensor of one dtype, the accumulators are fp32."""
    n = len(problems)
    descs = (_lib.VecGradDesc * n)()
    for d, pr in zip(descs, problems):
        dy = pr[0]
        _require_cuda(*pr)
        d.dy, d.ld, d.M, d.N = dy.data_ptr(), dy.stride(0), dy.shape[0], dy.shape[1]
        if len(pr) == 2:
            d.acc0 = pr[1].data_ptr()
        else:
            _, x, mean, rstd, dg, db = pr
            assert x.stride(0) == dy.stride(0)
            d.x, d.mean, d.rstd, d.acc0, d.acc1 = x.data_ptr(), mean.data_ptr(), rstd.data_ptr(), dg.data_ptr(), db.data_ptr()
    lib = _lib.load()
    dt = tp_dtype(problems[0][0].dtype)
    _lib.check(lib.tp_vec_param_grads(descs, n, dt, _stream()), "tp_vec_param_grads")
    _record("vec_param_grads", n, lambda s=None: lib.tp_vec_param_grads(descs, n, dt, _on(s)))


def accum_cast(dst, src_f32, accumulate):
    _require_cuda(dst, src_f32)
    lib = _lib.load()
    a = (_p(dst), _p(src_f32), dst.numel(), int(accumulate), tp_dtype(dst.dtype))
    _lib.check(lib.tp_accum_cast(*a, _stream()), "tp_accum_cast")
    _record("accum_cast", dst.numel(), lambda s=None: lib.tp_accum_cast(*a, _on(s)))
    return dst


def colsum_acc(x2d, acc_f32):
    _require_cuda(x2d, acc_f32)
    lib = _lib.load()
    a = (_p(x2d), x2d.stride(0), _p(acc_f32), x2d.shape[0], x2d.shape[1], tp_dtype(x2d.dtype))
    _lib.check(lib.tp_colsum_acc(*a, _stream()), "tp_colsum_acc")
    _record("colsum_acc", tuple(x2d.shape), lambda s=None: lib.tp_colsum_acc(*a, _on(s)))
    return acc_f32


def zero_(t):
    """Zero-fills a contiguous tensor whose byte size is a multiple of 4 with the library's fill kernel."""
    _require_cuda(t)
    nbytes = t.numel() * t.element_size()
    assert t.is_contiguous() and nbytes % 4 == 0
    lib = _lib.load()
    ptr = _p(t)
    _lib.check(lib.tp_zero_words(ptr, nbytes // 4, _stream()), "tp_zero_words")
    _record("zero", nbytes, lambda s=None: lib.tp_zero_words(ptr, nbytes // 4, _on(s)))
    return t


def fill_probe(big, small, hits_per_miss, workgroups, batches_per_wave, row_stride=0):
    """Launches the library's global -> LDS streaming probe (tp_fill_probe) on the current stream; returns the bytes
    it moves.  big / small: contiguous device tensors whose byte sizes are multiples of 8192.  row_stride (bytes):
    0 = consecutive bytes, else 64-row x 128-byte tiles of a matrix with that row pitch."""
    _require_cuda(big, small)
    lib = _lib.load()
    nb, ns = big.numel() * big.element_size(), small.numel() * small.element_size()
    _lib.check(lib.tp_fill_probe(_p(big), nb, _p(small), ns, int(hits_per_miss), int(workgroups), int(batches_per_wave),
                                 int(row_stride), _stream()), "tp_fill_probe")
    return workgroups * 4 * batches_per_wave * 8192


def embedding_fwd(ids, weight, out=None):
    """ids int64 [M] -> out [M, E] = weight[ids]."""
    _require_cuda(ids, weight)
    M, (V, E) = ids.numel(), weight.shape
    out = torch.empty(M, E, dtype=weight.dtype, device=weight.device) if out is None else out
    lib = _lib.load()
    _lib.check(lib.tp_embedding_fwd(_p(ids), _p(weight), _p(out), M, E, V, tp_dtype(weight.dtype), _stream()),
               "tp_embedding_fwd")
    return out


def embedding_bwd(ids, dout, dweight_acc):
    """dweight_acc fp32 [V, E] += scatter of dout [M, E] by ids."""
    _require_cuda(ids, dout, dweight_acc)
    V, E = dweight_acc.shape
    lib = _lib.load()
    _lib.check(lib.tp_embedding_bwd(_p(ids), _p(dout), _p(dweight_acc), ids.numel(), E, V, tp_dtype(dout.dtype),
                                    _stream()), "tp_embedding_bwd")
    return dweight_acc


def cross_entropy_(logits, target, V, grad_scale=1.0):
    """logits [M, Vpad] (row-major, first V columns valid) is overwritten with its gradient
    (softmax - onehot) * grad_scale; returns the per-row loss (fp32 [M])."""
    _require_cuda(logits, target)
    M, Vpad = logits.shape
    loss = torch.empty(M, dtype=torch.float32, device=logits.device)
    lib = _lib.load()
    _lib.check(lib.tp_cross_entropy(_p(logits), logits.stride(0), _p(target), _p(loss), M, V, Vpad, float(grad_scale),
                                    tp_dtype(logits.dtype), _stream()), "tp_cross_entropy")
    return loss


def scale_rows_(x2d, scale_f32):
    _require_cuda(x2d, scale_f32)
    lib = _lib.load()
    _lib.check(lib.tp_scale_rows(_p(x2d), x2d.stride(0), _p(scale_f32), x2d.shape[0], x2d.shape[1], tp_dtype(x2d.dtype),
                                 _stream()), "tp_scale_rows")
    return x2d
