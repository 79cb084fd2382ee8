"""ctypes binding of libterapipe_hip.so (the C ABI declared in include/terapipe_hip.h).

The library is loaded lazily and the load fails loudly: there is no CPU or PyTorch fallback for any
kernel.  If the shared object is missing it is built once with hipcc (``terapipe_amd.build``).
"""
import ctypes
import os
import threading

from . import build as _build

TP_F32, TP_F16, TP_BF16 = 0, 1, 2
TP_GEMM_NT, TP_GEMM_NN, TP_GEMM_TN = 0, 1, 2
(TP_EPI_STORE, TP_EPI_ACCUMULATE, TP_EPI_BIAS, TP_EPI_BIAS_RELU, TP_EPI_BIAS_GELU, TP_EPI_BIAS_RESIDUAL,
 TP_EPI_QKV_SCATTER, TP_EPI_RELU_GRAD, TP_EPI_GELU_GRAD) = range(9)

c_void_p, c_int, c_int32, c_int64, c_float, c_size_t = (
    ctypes.c_void_p, ctypes.c_int, ctypes.c_int32, ctypes.c_int64, ctypes.c_float, ctypes.c_size_t)


class GemmDesc(ctypes.Structure):
    """Mirror of ``tp_gemm_desc``."""
    _fields_ = [
        ("op", c_int32), ("dtype", c_int32), ("epilogue", c_int32),
        ("M", c_int32), ("N", c_int32), ("K", c_int32),
        ("A", c_void_p), ("lda", c_int64),
        ("B", c_void_p), ("ldb", c_int64),
        ("C", c_void_p), ("ldc", c_int64),
        ("bias", c_void_p),
        ("residual", c_void_p), ("ldr", c_int64),
        ("aux", c_void_p), ("ldaux", c_int64),
        ("aux_out", c_void_p), ("ldauxo", c_int64),
        ("colsum_acc", c_void_p),
        ("q", c_void_p), ("k_cache", c_void_p), ("v_cache", c_void_p),
        ("batch", c_int32), ("heads", c_int32), ("head_dim", c_int32), ("cache_len", c_int32),
        ("cache_rows", c_int64),
        ("q_scale", c_float), ("reserved", c_int32),
        ("q_bh_rows", c_int64),
        ("defer_reduce", c_int32), ("reserved4", c_int32),
    ]


class AttnDesc(ctypes.Structure):
    """Mirror of ``tp_attn_desc``."""
    _fields_ = [
        ("dtype", c_int32), ("batch", c_int32), ("heads", c_int32), ("head_dim", c_int32),
        ("T", c_int32), ("cache_len", c_int32),
        ("cache_rows", c_int64),
        ("q", c_void_p), ("k_cache", c_void_p), ("v_cache", c_void_p),
        ("o", c_void_p), ("lse", c_void_p),
        ("d_o", c_void_p), ("delta", c_void_p), ("dqkv", c_void_p),
        ("dk_cache", c_void_p), ("dv_cache", c_void_p),
        ("grad_cache_dtype", c_int32), ("accumulate_prefix", c_int32),
        ("has_incoming", c_int32), ("zero_slice_rows", c_int32),
        ("q_scale", c_float),
        ("colsum_dqkv_acc", c_void_p),
        ("reserved", c_int32), ("reserved2", c_int32),
        ("q_bh_rows", c_int64), ("stat_bh_rows", c_int64),
        ("dq_only", c_int32), ("reserved3", c_int32),
    ]


class AttnSuffixDesc(ctypes.Structure):
    """Mirror of ``tp_attn_suffix_desc``."""
    _fields_ = [
        ("dtype", c_int32), ("batch", c_int32), ("heads", c_int32), ("head_dim", c_int32),
        ("key_begin", c_int32), ("key_count", c_int32), ("q_end", c_int32), ("reserved", c_int32),
        ("cache_rows", c_int64), ("q_bh_rows", c_int64), ("stat_bh_rows", c_int64),
        ("k_cache", c_void_p), ("v_cache", c_void_p),
        ("q_all", c_void_p), ("d_o_all", c_void_p),
        ("lse_all", c_void_p), ("delta_all", c_void_p),
        ("dqkv", c_void_p),
    ]


class VecGradDesc(ctypes.Structure):
    """Mirror of ``tp_vecgrad_desc``."""
    _fields_ = [("dy", c_void_p), ("x", c_void_p), ("mean", c_void_p), ("rstd", c_void_p),
                ("acc0", c_void_p), ("acc1", c_void_p), ("ld", c_int64), ("M", c_int32), ("N", c_int32)]


class AdamTensor(ctypes.Structure):
    """Mirror of ``tp_adam_tensor``."""
    _fields_ = [("master", c_void_p), ("grad", c_void_p), ("exp_avg", c_void_p), ("exp_avg_sq", c_void_p),
                ("model", c_void_p), ("n", c_int64)]


class AdamDesc(ctypes.Structure):
    """Mirror of ``tp_adam_desc``."""
    _fields_ = [
        ("n_tensors", c_int32), ("grad_dtype", c_int32), ("model_dtype", c_int32), ("adam_w_mode", c_int32),
        ("bias_correction", c_int32), ("zero_grad", c_int32), ("step", c_int32), ("blocks_per_tensor", c_int32),
        ("lr", ctypes.c_double), ("beta1", ctypes.c_double), ("beta2", ctypes.c_double), ("eps", ctypes.c_double),
        ("weight_decay", ctypes.c_double), ("grad_scale", ctypes.c_double),
        ("tensors", c_void_p),
    ]


# every symbol include/terapipe_hip.h declares: name -> (restype, argtypes)
SYMBOLS = {
    "tp_version": (c_int, []),
    "tp_last_error": (ctypes.c_char_p, []),
    "tp_layernorm_fwd": (c_int, [c_void_p] * 6 + [c_int, c_int, c_float, c_int, c_void_p]),
    "tp_layernorm_bwd": (c_int, [c_void_p] * 11 + [c_int, c_int, c_int, c_void_p]),
    "tp_ln_param_grads": (c_int, [c_void_p] * 6 + [c_int, c_int, c_int, c_void_p]),
    "tp_layernorm_fwd_partials": (c_int, [c_void_p, c_int] + [c_void_p] * 8 + [c_int, c_int, c_float, c_int, c_void_p]),
    "tp_layernorm_bwd_partials": (c_int, [c_void_p, c_int] + [c_void_p] * 11 + [c_int, c_int, c_int, c_void_p]),
    "tp_vec_param_grads": (c_int, [ctypes.POINTER(VecGradDesc), c_int, c_int, c_void_p]),
    "tp_gemm_splits": (c_int, [ctypes.POINTER(GemmDesc)]),
    "tp_gemm_plan": (c_int, [ctypes.POINTER(GemmDesc), ctypes.POINTER(c_int), ctypes.POINTER(c_int)]),
    "tp_gemm_workspace_bytes": (c_size_t, [ctypes.POINTER(GemmDesc)]),
    "tp_gemm": (c_int, [ctypes.POINTER(GemmDesc), c_void_p, c_size_t, c_void_p]),
    "tp_gemm_static_ws_capacity": (c_size_t, []),
    "tp_gemm_static_ws": (c_int, [ctypes.POINTER(GemmDesc), c_void_p]),
    "tp_gemm_grouped": (c_int, [ctypes.POINTER(GemmDesc), c_int, c_void_p, c_size_t, c_void_p]),
    "tp_gemm_group_cfg": (c_int, [ctypes.POINTER(GemmDesc), c_int]),
    "tp_attn_fwd_workspace_bytes": (c_size_t, [ctypes.POINTER(AttnDesc)]),
    "tp_attn_prefix_fwd": (c_int, [ctypes.POINTER(AttnDesc), c_void_p, c_size_t, c_void_p]),
    "tp_attn_bwd_workspace_bytes": (c_size_t, [ctypes.POINTER(AttnDesc)]),
    "tp_attn_prefix_bwd": (c_int, [ctypes.POINTER(AttnDesc), c_void_p, c_size_t, c_void_p]),
    "tp_attn_suffix_dkdv": (c_int, [ctypes.POINTER(AttnSuffixDesc), c_void_p]),
    "tp_attn_bwd_fused": (c_int, [ctypes.POINTER(AttnDesc), ctypes.POINTER(AttnSuffixDesc), c_void_p, c_int, c_void_p]),
    "tp_embedding_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "tp_embedding_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "tp_cross_entropy": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_int, c_void_p]),
    "tp_scale_rows": (c_int, [c_void_p, c_int64, c_void_p, c_int, c_int, c_int, c_void_p]),
    "tp_plan_slices": (c_int, [c_void_p, c_int, c_int, c_int, ctypes.c_double] + [c_void_p] * 5),
    "tp_adam_check_table": (c_int, [c_void_p, c_int, c_int]),
    "tp_adam_step": (c_int, [ctypes.POINTER(AdamDesc), c_void_p]),
    "tp_accum_cast": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "tp_colsum_acc": (c_int, [c_void_p, c_int64, c_void_p, c_int, c_int, c_int, c_void_p]),
    "tp_zero_words": (c_int, [c_void_p, c_int64, c_void_p]),
    "tp_fill_probe": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int, c_int, c_int, c_int64, c_void_p]),
}

_lock = threading.Lock()
_lib = None


class TeraPipeHipError(RuntimeError):
    pass


def lib_path():
    return _build.LIB_PATH


def load(build_if_missing=True):
    """Returns the loaded library; builds it first if the .so is not there.  Raises on any failure."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = lib_path()
        if not os.path.exists(path):
            if not build_if_missing:
                raise TeraPipeHipError("%s is missing; run `python -m terapipe_amd.build`" % path)
            _build.build(verbose=False)
        lib = ctypes.CDLL(path)
        for name, (restype, argtypes) in SYMBOLS.items():
            fn = getattr(lib, name)  # AttributeError if the export is missing
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def check(rc, what=""):
    if rc != 0:
        msg = load().tp_last_error()
        raise TeraPipeHipError("%s failed with status %d: %s" % (what or "libterapipe_hip", rc, (msg or b"").decode()))
