"""Writes tests/golden/c1_tiny_fp32.npz: sub-sampled outputs and gradients of the oracle on the tiny
fp32 config (4 layers, hidden 256, 4 heads, FFN 1024, seq 128, batch 2, 8 slices of 16).  The vectors
come from the oracle itself (the reference ships no fixtures for this path and is not imported); they
are a drift guard, not the oracle's proof -- that is tests/test_oracle_pins.py."""
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
import oracle  # noqa: E402

cfg = dict(n_layers=4, E=256, H=4, F=1024, L=128, B=2, n_slices=8, seed=0)
ps = oracle.init_stack_params(cfg["n_layers"], cfg["E"], cfg["F"], 0.02, torch.float32, seed=cfg["seed"])
g = torch.Generator().manual_seed(cfg["seed"] + 1)
x = torch.randn(cfg["L"], cfg["B"], cfg["E"], generator=g)
dy = torch.randn(cfg["L"], cfg["B"], cfg["E"], generator=g)
leaf = [{k: v.clone().requires_grad_(True) for k, v in p.items()} for p in ps]
y, dx, fc = oracle.terapipe_forward_backward(leaf, x, dy, cfg["H"], [cfg["B"]],
                                             oracle.uniform_slice(cfg["L"], cfg["n_slices"]))
out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c1_tiny_fp32.npz")
np.savez_compressed(out, y_sub=y[::7, :, ::5].numpy(), dx_sub=dx[::7, :, ::5].numpy(),
                    dfc1_sub=leaf[0]["fc1.weight"].grad[::16, ::8].numpy(),
                    dbqkv3=leaf[3]["attn.in_proj.bias"].grad.numpy(),
                    vcache0_sub=fc[0][1][::3, ::9, ::4].numpy(), **{k: np.int64(v) for k, v in cfg.items()})
print("wrote", out, os.path.getsize(out), "bytes")
