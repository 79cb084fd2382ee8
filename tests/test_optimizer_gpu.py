"""Optimizer step (tp_adam_step through terapipe_amd.FusedAdam) against the oracle's float64 restatement of
the reference's update_weights (test_transformer_terapipe.py:245-266), and against torch.optim on the GPU.
Tolerance: fp32 state within 1e-5 of max|ref| after several steps; the 16-bit model copy is bit-exact to the
rounded master."""
import numpy as np
import pytest
import torch

from oracle import optimizer_oracle as opt

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SIZES = [1, 3, 1027, 4096, 70001]


def _rel(a, ref):
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.max(np.abs(a.double().cpu().numpy().reshape(-1) - ref.reshape(-1))) / max(np.max(np.abs(ref)), 1e-30))


@pytest.mark.parametrize("adam_w_mode,wd,bias_correction", [(True, 0.0, True), (False, 0.05, True), (True, 0.05, True),
                                                            (True, 0.0, False)])
def test_step_fp32_matches_oracle(adam_w_mode, wd, bias_correction):
    from terapipe_amd import FusedAdam
    g = torch.Generator().manual_seed(5)
    params = [torch.randn(n, generator=g).to(DEV).requires_grad_() for n in SIZES]
    ref = [(p.detach().double().cpu().numpy(), np.zeros(p.numel()), np.zeros(p.numel())) for p in params]
    hyper = dict(lr=2e-3, beta1=0.85, beta2=0.97, eps=1e-7, weight_decay=wd)
    o = FusedAdam(params, lr=hyper["lr"], betas=(hyper["beta1"], hyper["beta2"]), eps=hyper["eps"], weight_decay=wd,
                  adam_w_mode=adam_w_mode, bias_correction=bias_correction)
    for step in range(1, 6):
        for i, p in enumerate(params):
            gr = torch.randn(p.numel(), generator=g) * step
            p.grad = gr.to(DEV)
            ref[i] = opt.adam_step(ref[i][0], gr.double().numpy(), ref[i][1], ref[i][2], step,
                                   adam_w_mode=adam_w_mode, bias_correction=bias_correction, **hyper)
        o.step()
        for i, p in enumerate(params):
            assert _rel(p.detach(), ref[i][0]) <= 1e-5, (step, SIZES[i])
            assert _rel(o.state[p]["exp_avg"], ref[i][1]) <= 1e-5
            assert _rel(o.state[p]["exp_avg_sq"], ref[i][2]) <= 1e-5
    o.zero_grad()
    assert all(p.grad is None for p in params)


def test_step_matches_torch_adam_on_gpu():
    from terapipe_amd import FusedAdam
    g = torch.Generator().manual_seed(9)
    a = [torch.randn(4, 515, generator=g).to(DEV).requires_grad_() for _ in range(3)]
    b = [p.detach().clone().requires_grad_() for p in a]
    oa = FusedAdam(a, lr=1e-2, weight_decay=0.0)
    ob = torch.optim.Adam(b, lr=1e-2)
    for step in range(4):
        for p, q in zip(a, b):
            p.grad = torch.randn(4, 515, generator=g).to(DEV)
            q.grad = p.grad.clone()
        oa.step()
        ob.step()
    for p, q in zip(a, b):
        assert _rel(p.detach(), q.detach().double().cpu().numpy()) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("zero_grads", [False, True])
def test_update_weights_mixed_precision(dtype, zero_grads):
    """fp16/bf16 model parameters with loss-scaled 16-bit gradients, fp32 master weights (:92-95, :245-266)."""
    from terapipe_amd import FusedAdam
    g = torch.Generator().manual_seed(3)
    shapes = [(64, 48), (48,), (1, 5), (129, 7)]
    model = [(torch.randn(*s, generator=g) * 0.02).to(dtype).to(DEV).requires_grad_() for s in shapes]
    master = [p.detach().clone().float() for p in model]          # :92
    ref = [(m.double().cpu().numpy().reshape(-1), np.zeros(m.numel()), np.zeros(m.numel())) for m in master]
    o = FusedAdam(master, lr=1e-3)
    scale = 128.0
    for step in range(1, 5):
        grads = []
        for i, p in enumerate(model):
            gr = (torch.randn(*shapes[i], generator=g) * scale * 0.1).to(dtype)
            p.grad = gr.to(DEV)
            grads.append(p.grad)
            ref[i] = opt.adam_step(ref[i][0], gr.double().numpy().reshape(-1), ref[i][1], ref[i][2], step, lr=1e-3,
                                   grad_scale=1.0 / scale)
        o.update_weights(model, loss_scale=scale, zero_grads=zero_grads)
        for i, p in enumerate(model):
            assert _rel(master[i], ref[i][0]) <= 1e-5
            assert _rel(o.state[master[i]]["exp_avg_sq"], ref[i][2]) <= 1e-5
            assert torch.equal(p.detach(), master[i].to(dtype))                 # :262-266 model_param.copy_(master)
            if zero_grads:
                assert p.grad.data_ptr() == grads[i].data_ptr() and not bool(p.grad.any())
            else:
                assert p.grad is None                                           # :253 del model_param.grad


def test_errors():
    from terapipe_amd import FusedAdam, _lib
    p = torch.zeros(64, device=DEV)
    with pytest.raises(RuntimeError):
        FusedAdam([p], amsgrad=True)
    q = torch.zeros(65, device=DEV)[1:].requires_grad_()                        # 4-byte aligned only
    q.grad = torch.ones(65, device=DEV)[1:]
    with pytest.raises(_lib.TeraPipeHipError, match="aligned"):
        FusedAdam([q]).step()
    h = torch.zeros(8, device=DEV, dtype=torch.float16).requires_grad_()
    h.grad = torch.ones_like(h)
    with pytest.raises(TypeError):
        FusedAdam([h]).step()
    with pytest.raises(ValueError):
        FusedAdam([p]).update_weights([h, h])
