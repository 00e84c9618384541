"""`generalized_delta_rule_resets`: a padded batch with per-row lengths and in-row resets (the `length` and
`new_starts` of the reference's XLA-FFI kernel, /root/reference/rwkv_ops/rwkv7_kernel/cuda_kernel/wkv7_jax.cu:18,
23-24,46-51,66) against the CPU oracle run document by document."""
import pytest
import torch

import rwkv_ops_amd
from oracle import rwkv7_native as orc
from rwkv_ops_amd.synthetic import GRAD_TOL, make_inputs, rel_l2

pytestmark = pytest.mark.gpu


def reference(xs, h0, length, new_starts):
    """The loop of wkv7_jax.cu:36-66 in terms of the oracle: reset where flagged, hand back the state after token
    length - 1; outputs only for the valid tokens (the rest is padding)."""
    B, T = xs[0].shape[:2]
    o = torch.zeros(xs[0].shape, dtype=torch.float32)
    states = []
    for b in range(B):
        state = h0[b:b + 1].clone()
        n = length[b]
        cuts = sorted({0, n} | {t for t in range(1, n) if new_starts[b][t]})
        if new_starts[b][0]:
            state = torch.zeros_like(state)
        for t0, t1 in zip(cuts, cuts[1:]):
            if t0 > 0 and new_starts[b][t0]:
                state = torch.zeros_like(state)
            ob, state = orc.generalized_delta_rule(*[x[b:b + 1, t0:t1].float() for x in xs], state)
            o[b:b + 1, t0:t1] = ob
        states.append(state)
    return o, torch.cat(states)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 5e-3)])
def test_lengths_and_resets_match_the_oracle(device, dtype, tol):
    B, T, H = 4, 150, 2
    xs = make_inputs(B, T, H, 64, seed=9900, dtype=dtype)
    length = [150, 97, 0, 64]
    ns = [[False] * T for _ in range(B)]
    ns[0][70] = True                       # two documents in row 0
    ns[1][0] = True                        # row 1 does not take its initial state
    ns[1][33] = ns[1][34] = True           # a one-token document
    ns[3][64] = True                       # a reset exactly where the row's valid part ends
    o, s = rwkv_ops_amd.generalized_delta_rule_resets(*[x.to(device) for x in xs[:6]], initial_state=xs[6].to(device),
                                                      length=length, new_starts=torch.tensor(ns))
    assert o.shape == xs[0].shape and o.dtype == dtype and s.shape == xs[6].shape and s.dtype == torch.float32
    o_ref, s_ref = reference(xs[:6], xs[6], length, ns)
    for b in range(B):
        n = length[b]
        if n:
            assert rel_l2(o[b, :n], o_ref[b, :n]) < (tol if n * H * 64 >= 4096 else 2 * tol), b
        assert rel_l2(s[b], s_ref[b]) < tol, b
    assert torch.equal(s[2].cpu(), xs[6][2])      # no valid token: the state the row started from


def test_gradients_flow_through_the_wrapper(device):
    B, T, H = 2, 130, 2
    xs = make_inputs(B, T, H, 64, seed=9901, dtype=torch.bfloat16)
    length = [130, 80]
    ns = [[False] * T for _ in range(B)]
    ns[0][50] = True
    g = torch.Generator().manual_seed(3)
    dO = torch.randn(B, T, H, 64, generator=g).to(torch.bfloat16)
    dO[1, 80:] = 0                                 # the padding takes no gradient
    dS = 0.1 * torch.randn(B, H, 64, 64, generator=g)
    leaves = [x.to(device).requires_grad_(True) for x in xs[:6]]
    h0 = xs[6].to(device).requires_grad_(True)
    o, s = rwkv_ops_amd.generalized_delta_rule_resets(*leaves, initial_state=h0, length=length, new_starts=ns)
    loss = (o.float() * dO.to(device).float()).sum() + (s * dS.to(device)).sum()
    got = torch.autograd.grad(loss, leaves + [h0])
    # the same through autograd over the oracle, document by document
    ref_leaves = [x.float().clone().requires_grad_(True) for x in xs[:6]]
    ref_h0 = xs[6].clone().requires_grad_(True)
    total = 0
    for b in range(B):
        state = ref_h0[b:b + 1]
        n = length[b]
        cuts = sorted({0, n} | {t for t in range(1, n) if ns[b][t]})
        for t0, t1 in zip(cuts, cuts[1:]):
            if t0 > 0 and ns[b][t0]:
                state = torch.zeros_like(state)
            ob, state = orc.generalized_delta_rule(*[x[b:b + 1, t0:t1] for x in ref_leaves], state)
            total = total + (ob * dO[b:b + 1, t0:t1].float()).sum()
        total = total + (state * dS[b:b + 1]).sum()
    ref = torch.autograd.grad(total, ref_leaves + [ref_h0])
    for name, a_, b_ in zip(("dr", "dw", "dk", "dv", "da", "db", "dh0"), got, ref):
        assert rel_l2(a_, b_) < GRAD_TOL[name], (name, rel_l2(a_, b_))
