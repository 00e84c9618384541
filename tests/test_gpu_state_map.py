"""Initial states gathered through ``state_map`` (GPU): every forward path, the decode pool and the
gradient of the shared states, against the CPU oracle run on the gathered states.

The oracle itself has no state_map: the test gathers ``pool[state_map]`` for it (and scatters the
gradient back with ``index_add_``), which is the definition of the feature
(/root/reference/rwkv_ops/rwkv6_kernel/ops_rwkv_kernel.py:57 ``ops.take(init_state, state_map, axis=0)``)."""
import pytest
import torch

import rwkv_ops_amd
from oracle import rwkv7_native as orc
from rwkv_ops_amd.synthetic import make_inputs, rel_l2

pytestmark = pytest.mark.gpu


def _pool(n_state, H, seed):
    g = torch.Generator().manual_seed(seed)
    return 0.1 * torch.randn(n_state, H, 64, 64, generator=g)


# fp32 recurrent path, two-kernel bf16 path (B*H < 72), fused bf16 path, T = 1 (decode kernel)
@pytest.mark.parametrize("B,T,H,dtype,tol", [(3, 70, 2, torch.float32, 1e-4), (3, 130, 4, torch.bfloat16, 5e-3),
                                             (4, 130, 32, torch.bfloat16, 5e-3), (5, 1, 3, torch.bfloat16, 5e-3)])
def test_forward_with_state_map(device, B, T, H, dtype, tol):
    xs = make_inputs(B, T, H, 64, seed=300 + T, dtype=dtype)
    pool = _pool(B + 2, H, seed=T)
    smap = [(2 * i + 1) % (B + 2) for i in range(B)]
    smap[-1] = smap[0]                                   # two rows share a state
    o_ref, s_ref = orc.generalized_delta_rule(*[x.float() for x in xs[:6]], pool[smap])
    dev = [x.to(device) for x in xs[:6]]
    for m in (smap, torch.tensor(smap, dtype=torch.int64, device=device)):
        o, s = rwkv_ops_amd.generalized_delta_rule(*dev, initial_state=pool.to(device), state_map=m)
        assert s.shape == (B, H, 64, 64)
        eo, es = rel_l2(o, o_ref), rel_l2(s, s_ref)
        print(f"B={B} T={T} H={H} {dtype}: rel_l2 o={eo:.2e} state={es:.2e}")
        assert eo < tol and es < tol
    # identical to passing the gathered states
    o2, s2 = rwkv_ops_amd.generalized_delta_rule(*dev, initial_state=pool[smap].to(device))
    assert torch.equal(o.cpu(), o2.cpu()) and torch.equal(s.cpu(), s2.cpu())


def test_state_map_validation(device):
    xs = [x.to(device) for x in make_inputs(2, 8, 2, 64, seed=1, dtype=torch.bfloat16)]
    pool = _pool(3, 2, 0).to(device)
    with pytest.raises(ValueError):
        rwkv_ops_amd.generalized_delta_rule(*xs[:6], initial_state=pool, state_map=[0, 3])      # out of range
    with pytest.raises(ValueError):
        rwkv_ops_amd.generalized_delta_rule(*xs[:6], initial_state=pool, state_map=[0, 1, 2])   # wrong length
    with pytest.raises(ValueError):
        rwkv_ops_amd.generalized_delta_rule(*xs[:6], initial_state=pool)                        # 3 states, 2 rows, no map


def test_backward_scatters_state_gradient(device):
    B, T, H = 3, 100, 2
    xs = make_inputs(B, T, H, 64, seed=77, dtype=torch.bfloat16)
    pool = _pool(2, H, 5)
    smap = [1, 0, 1]
    g = torch.Generator().manual_seed(9)
    dO = torch.randn(B, T, H, 64, generator=g).to(torch.bfloat16)
    dS = 0.1 * torch.randn(B, H, 64, 64, generator=g)
    ref = orc.gradients(*xs[:6], pool[smap], dO, dS)
    dpool_ref = torch.zeros_like(pool).index_add_(0, torch.tensor(smap), ref[6])
    leaves = [x.to(device).requires_grad_(True) for x in xs[:6]]
    p = pool.to(device).requires_grad_(True)
    o, s = rwkv_ops_amd.generalized_delta_rule(*leaves, initial_state=p, state_map=smap)
    loss = (o.float() * dO.to(device).float()).sum() + (s * dS.to(device)).sum()
    got = torch.autograd.grad(loss, leaves + [p])
    for name, a_, b_ in zip(["dr", "dw", "dk", "dv", "da", "db"], got[:6], ref[:6]):
        assert rel_l2(a_, b_) < 1e-2, name
    e = rel_l2(got[6], dpool_ref)
    print(f"d(pool): {e:.2e}")
    assert got[6].shape == pool.shape and e < 6e-3


def test_decode_pool_in_place(device):
    B, H, n_state, steps = 4, 3, 7, 3
    xs = make_inputs(B, steps, H, 64, seed=11, dtype=torch.bfloat16)
    pool = _pool(n_state, H, 3)
    smap = [5, 0, 3, 6]
    dpool = pool.to(device).clone()
    state_ref = pool[smap].clone()
    for t in range(steps):
        step = [x[:, t:t + 1] for x in xs[:6]]
        o_ref, state_ref = orc.generalized_delta_rule(*[x.float() for x in step], state_ref)
        o = rwkv_ops_amd.rwkv7_decode_step(*[x[:, t].to(device) for x in xs[:6]], dpool,
                                           state_map=torch.tensor(smap, dtype=torch.int32, device=device))
        assert rel_l2(o, o_ref[:, 0]) < 5e-3
    got = dpool.cpu()
    assert rel_l2(got[smap], state_ref) < 1e-5
    untouched = [i for i in range(n_state) if i not in smap]
    assert torch.equal(got[untouched], pool[untouched])          # other slots: bitwise unchanged
    with pytest.raises(ValueError):
        rwkv_ops_amd.rwkv7_decode_step(*[x[:, 0].to(device) for x in xs[:6]], dpool, state_map=[1, 1, 2, 3])


def test_a_bad_device_map_does_not_fault(device):
    """A map that arrives on the device is never read back, so nothing checks it: the kernels clamp what they read,
    and the backward's gather and scatter on the host side clamp the same way (no device-side index assertion)."""
    B, T, H, n_state = 3, 70, 2, 4
    xs = make_inputs(B, T, H, 64, seed=411, dtype=torch.bfloat16)
    pool = _pool(n_state, H, seed=5)
    bad = torch.tensor([-3, 2, 99], dtype=torch.int32, device=device)
    good = bad.clamp(0, n_state - 1)
    outs = []
    for m in (bad, good):
        dev = [x.to(device).requires_grad_(True) for x in xs[:6]]
        p = pool.to(device).requires_grad_(True)
        o, s = rwkv_ops_amd.generalized_delta_rule(*dev, initial_state=p, state_map=m)
        (o.float().sum() + s.sum()).backward()
        torch.cuda.synchronize()
        outs.append([o, s, p.grad] + [d.grad for d in dev])
    for x, y in zip(*outs):
        assert torch.equal(x, y)
