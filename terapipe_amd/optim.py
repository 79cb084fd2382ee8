"""Optimizer step of the reference's training loop on the HIP path.

``FusedAdam`` has the constructor and ``step`` / ``zero_grad`` surface of ``apex.optimizers.FusedAdam`` as the
reference uses it (test_transformer_terapipe.py:92-97: fp32 master copies of the parameters, ``lr=1e-10``).
``step`` runs one ``tp_adam_step`` launch per (gradient dtype, model dtype) group over a device table of tensor
records.  ``update_weights`` is the reference's whole mixed-precision update (:245-266) in that one launch: the
16-bit gradients are read directly and multiplied by 1/loss-scale, the fp32 master weights and moments are
updated, the 16-bit model weights are rewritten and the gradients dropped.
"""
import ctypes

import torch

from . import _lib
from .ops import _record, _stream, tp_dtype


class FusedAdam(torch.optim.Optimizer):
    def __init__(self, params, lr=1e-3, bias_correction=True, betas=(0.9, 0.999), eps=1e-8, adam_w_mode=True,
                 weight_decay=0.0, amsgrad=False, set_grad_none=True):
        if amsgrad:
            raise RuntimeError("FusedAdam does not support the AMSGrad variant.")     # as apex raises
        defaults = dict(lr=lr, bias_correction=bias_correction, betas=betas, eps=eps, weight_decay=weight_decay)
        super().__init__(params, defaults)
        self.adam_w_mode = 1 if adam_w_mode else 0
        self.set_grad_none = set_grad_none
        self.blocks_per_tensor = 0  # 0 = the library's default
        self._tables = {}           # (pointer tuple, device table) per launch group: re-uploaded only when a
                                    # tensor moved (gradients released after each step get new addresses)

    def zero_grad(self, set_to_none=None):
        if set_to_none is None:
            set_to_none = self.set_grad_none
        for group in self.param_groups:
            for p in group["params"]:
                if p.grad is None:
                    continue
                if set_to_none:
                    p.grad = None
                else:
                    p.grad.zero_()

    def _state_of(self, p):
        st = self.state[p]
        if len(st) == 0:
            st["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
            st["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
        return st

    def _launch(self, group, records, grad_dtype, model_dtype, grad_scale, zero_grad, key):
        """records: list of (master, grad, model or None)."""
        n = len(records)
        host = (_lib.AdamTensor * n)()
        for i, (p, g, w) in enumerate(records):
            st = self._state_of(p)
            for t in (p, g, st["exp_avg"], st["exp_avg_sq"]) + ((w,) if w is not None else ()):
                if not t.is_cuda or not t.is_contiguous():
                    raise ValueError("FusedAdam needs contiguous tensors on the GPU")
            if p.dtype != torch.float32:
                raise TypeError("FusedAdam updates fp32 weights (got %s); keep fp32 master copies of 16-bit "
                                "parameters and call update_weights" % p.dtype)
            if g.numel() != p.numel() or (w is not None and w.numel() != p.numel()):
                raise ValueError("gradient / model tensor size differs from the master weight's")
            host[i].master, host[i].grad = p.data_ptr(), g.data_ptr()
            host[i].exp_avg, host[i].exp_avg_sq = st["exp_avg"].data_ptr(), st["exp_avg_sq"].data_ptr()
            host[i].model = w.data_ptr() if w is not None else None
            host[i].n = p.numel()
        lib = _lib.load()
        md = tp_dtype(model_dtype) if model_dtype is not None else -1
        _lib.check(lib.tp_adam_check_table(ctypes.cast(host, ctypes.c_void_p), n, md), "tp_adam_check_table")
        image = bytes(host)
        cached = self._tables.get(key)
        if cached is not None and cached[0] == image:
            table = cached[1]
        else:
            table = torch.frombuffer(bytearray(image), dtype=torch.uint8).to(records[0][0].device, non_blocking=False)
            self._tables[key] = (image, table)
        d = _lib.AdamDesc()
        d.n_tensors, d.grad_dtype, d.model_dtype = n, tp_dtype(grad_dtype), md
        d.adam_w_mode, d.bias_correction = self.adam_w_mode, 1 if group["bias_correction"] else 0
        d.zero_grad, d.step, d.blocks_per_tensor = 1 if zero_grad else 0, group["step"], self.blocks_per_tensor
        d.lr, (d.beta1, d.beta2), d.eps = group["lr"], group["betas"], group["eps"]
        d.weight_decay, d.grad_scale = group["weight_decay"], grad_scale
        d.tensors = table.data_ptr()
        elems = sum(r[0].numel() for r in records)

        def run(stream=None):
            _lib.check(lib.tp_adam_step(ctypes.byref(d), _stream() if stream is None else stream), "tp_adam_step")
        _record("adam", dict(elems=elems, grad_bytes=torch.empty(0, dtype=grad_dtype).element_size(),
                             model_bytes=0 if model_dtype is None else 2, zero_grad=bool(zero_grad)), run)
        run()

    def _step_groups(self, model_params, grad_scale, zero_grad):
        models = None
        if model_params is not None:
            models = list(model_params)
            n_master = sum(len(g["params"]) for g in self.param_groups)
            if len(models) != n_master:
                raise ValueError("update_weights: %d model parameters for %d master parameters" % (len(models), n_master))
        pos = 0
        for gi, group in enumerate(self.param_groups):
            group["step"] = group.get("step", 0) + 1
            buckets = {}
            for p in group["params"]:
                w = models[pos] if models is not None else None
                pos += 1
                g = (w.grad if w is not None else p.grad)
                if g is None:
                    continue
                if g.is_sparse:
                    raise RuntimeError("FusedAdam does not support sparse gradients")
                key = (g.dtype, w.dtype if w is not None else None, p.device)
                buckets.setdefault(key, []).append((p, g, w))
            for key, records in buckets.items():
                with torch.cuda.device(key[2]):
                    self._launch(group, records, key[0], key[1], grad_scale, zero_grad, (gi,) + key)

    @torch.no_grad()
    def step(self, closure=None):
        """One Adam update of the (fp32) parameters from their ``.grad`` (apex FusedAdam.step)."""
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        self._step_groups(None, 1.0, False)
        return loss

    @torch.no_grad()
    def update_weights(self, model_params, loss_scale=1.0, zero_grads=False):
        """The reference's mixed-precision ``update_weights`` (test_transformer_terapipe.py:245-266) in one pass:
        ``model_params`` are the 16-bit parameters, in the order of the fp32 master parameters this optimizer
        was built on; their ``.grad`` (scaled by ``loss_scale``) drives the update, the new master weights are
        written back to them, and their gradients are released (``del model_param.grad``, :253) or, with
        ``zero_grads``, kept and zeroed in the same pass."""
        models = list(model_params)
        self._step_groups(models, 1.0 / float(loss_scale), bool(zero_grads))
        if not zero_grads:
            for w in models:
                w.grad = None
