"""Seeded synthetic inputs with the distributions the benchmark configurations name.

r, k, v ~ N(0, 1); the ``w`` argument is ``-exp(-softplus(-x) - 0.5)`` with x ~ N(0, 1)
(the operator applies ``exp(-exp(w))`` to it, as every path of the reference does:
/root/reference/rwkv_ops/rwkv7_kernel/native_keras_op.py:58,
/root/reference/rwkv_ops/rwkv7_kernel/torch_op.py:433-434); kappa is a per-head
L2-normalised N(0, 1) vector, a = -kappa, b = kappa * sigmoid(y), y ~ N(0, 1)
(the construction of /root/reference/test_script/test_rwkv7_value.py:36-45,80-82);
the initial state is 0.1 * N(0, 1), float32, ``[B, H, K, V]``.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def make_inputs(B, T, H, N=64, *, seed=0, dtype=torch.float32, h0=True, h0_batch=None,
                device="cpu"):
    """Returns ``(r, w, k, v, a, b, h0)``.  Values are drawn in float32 on the CPU from
    ``seed`` and rounded once to ``dtype``; ``h0`` stays float32 (or None)."""
    g = torch.Generator(device="cpu").manual_seed(int(seed))

    def randn(*shape):
        return torch.randn(*shape, generator=g, dtype=torch.float32)

    r, k, v = randn(B, T, H, N), randn(B, T, H, N), randn(B, T, H, N)
    w = -torch.exp(-F.softplus(-randn(B, T, H, N)) - 0.5)
    kappa = F.normalize(randn(B, T, H, N), dim=-1, eps=1e-12)
    a = -kappa
    b = kappa * torch.sigmoid(randn(B, T, H, N))
    state = None
    if h0:
        state = 0.1 * randn(B if h0_batch is None else h0_batch, H, N, N)
        state = state.to(device)
    r, w, k, v, a, b = (x.to(dtype).to(device) for x in (r, w, k, v, a, b))
    return r, w, k, v, a, b, state


# Relative-L2 thresholds of the bf16 backward against float32 autograd through the oracle on the same rounded
# inputs, per gradient (the reference states none).  Largest values measured over the GPU tests: dr 3.3e-3,
# dw 3.5e-3, dk 3.7e-3, dv 3.7e-3, dh0 3.2e-3; da 5.4e-3 and db 5.9e-3 (the latter on a single 64-token chunk of one
# head, 5.1e-3 otherwise; 4.7e-3 at the training shape): these two pass through the triangular inverse and its
# adjoint, two more bf16 roundings than the others.
GRAD_NAMES = ("dr", "dw", "dk", "dv", "da", "db", "dh0")
GRAD_TOL = {"dr": 5e-3, "dw": 5e-3, "dk": 5e-3, "dv": 5e-3, "da": 6e-3, "db": 6e-3, "dh0": 5e-3}


def rel_l2(x, ref):
    """Relative L2 error ``|x - ref| / |ref|`` in float64 (the parity metric)."""
    x = x.detach().double().cpu()
    ref = ref.detach().double().cpu()
    den = ref.norm()
    return float((x - ref).norm() / den) if den > 0 else float((x - ref).norm())
