"""CPU restatement of the reference's optimizer step (test_transformer_terapipe.py:245-266 around apex's
FusedAdam, :95) in numpy.  TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).  apex is not in this image; its
published update (multi_tensor_adam: L2 mode adds wd*p to the gradient, AdamW mode adds wd*p to the update)
is restated here and pinned in tests/test_oracle_pins.py against the library routines torch.optim.Adam
(L2 mode) and torch.optim.AdamW (decoupled mode) on the CPU, over several steps so that a wrong bias
correction, moment coefficient or decay placement shows."""
import numpy as np


def adam_step(p, g, m, v, step, lr, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0, adam_w_mode=True,
              bias_correction=True, grad_scale=1.0):
    """One update of float64 arrays; returns (p, m, v).  ``step`` counts from 1."""
    p, g, m, v = (np.asarray(a, dtype=np.float64) for a in (p, g, m, v))
    g = g * grad_scale                                     # :252 mul_(1 / LOSS_SCALE_FACTOR)
    if not adam_w_mode:
        g = g + weight_decay * p
    m = beta1 * m + (1.0 - beta1) * g
    v = beta2 * v + (1.0 - beta2) * g * g
    bc1 = 1.0 - beta1 ** step if bias_correction else 1.0
    bc2 = 1.0 - beta2 ** step if bias_correction else 1.0
    update = (m / bc1) / (np.sqrt(v / bc2) + eps)
    if adam_w_mode:
        update = update + weight_decay * p
    return p - lr * update, m, v


def update_weights(master, model_grad, m, v, step, loss_scale, model_dtype, **hyper):
    """Mixed-precision update (:245-266): returns (master, m, v, model) with model = master rounded to
    ``model_dtype`` (a numpy dtype, or a callable that rounds float64 to the 16-bit format)."""
    master, m, v = adam_step(master, model_grad, m, v, step, grad_scale=1.0 / loss_scale, **hyper)
    master32 = master.astype(np.float32)
    model = model_dtype(master32) if callable(model_dtype) else master32.astype(model_dtype)
    return master, m, v, model
