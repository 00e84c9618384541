"""A seeded sweep over random shapes, decay regimes and call variants (GPU): forward against the C oracle
(dense batches, packed sequences, the RWKV6 operator),
a few small cases backward against autograd through the torch oracle.  Tolerances as in the other GPU tests
(5e-3 relative L2 forward; the per-gradient thresholds of tests/test_gpu_backward.py)."""
import random

import pytest
import torch

import rwkv_ops_amd
from oracle import native_c
from oracle import rwkv7_native as orc
from rwkv_ops_amd.synthetic import make_inputs, rel_l2
from tests.test_gpu_backward import check, grads_gpu

pytestmark = pytest.mark.gpu
TOL = 5e-3


def _decays(kind, shape, g):
    if kind == "model":        # RWKV7's own parameterisation, as in the benchmark inputs
        return None
    if kind == "normal":       # what the reference's smoke test feeds: several exponent buckets per chunk
        return torch.randn(shape, generator=g)
    if kind == "slow":         # decay factors close to one
        return -5.0 + torch.randn(shape, generator=g)
    if kind == "mixed":
        return 3.0 * torch.randn(shape, generator=g) - 1.0
    # per-channel regimes: some channels forget at once, some never
    base = torch.tensor([-8.0, -2.0, 0.0, 2.0])[torch.randint(0, 4, (shape[-1],), generator=g)]
    return base + 0.3 * torch.randn(shape, generator=g)


def _cases():
    rnd = random.Random(20240611)
    out = []
    for i in range(28):
        big = i % 4 == 3                                   # one-kernel form (B*H >= 96)
        B = rnd.randint(1, 4)
        H = rnd.randint(96 // B + 1, 160 // B) if big else rnd.randint(1, max(1, 95 // B))
        T = rnd.choice([1, 2, 15, 63, 64, 65, 127, 128, 129]) if i % 7 == 0 else rnd.randint(1, 200 if big else 420)
        out.append((i, B, T, H, rnd.choice(["model", "model", "normal", "slow", "mixed", "channels"]),
                    rnd.choice(["given", "given", "none", "shared"]), rnd.random() < 0.25))
    return out


@pytest.mark.parametrize("i,B,T,H,decay,state,head_first", _cases())
def test_random_forward(device, i, B, T, H, decay, state, head_first):
    xs = list(make_inputs(B, T, H, 64, seed=7000 + i, dtype=torch.bfloat16,
                          h0=state != "none", h0_batch=1 if state == "shared" else None))
    g = torch.Generator().manual_seed(i)
    w = _decays(decay, (B, T, H, 64), g)
    if w is not None:
        xs[1] = w.to(torch.bfloat16)
    o_ref, s_ref = native_c.run(*xs[:6], xs[6])
    dev = [None if x is None else x.to(device) for x in xs]
    if head_first:
        dev[:6] = [x.permute(0, 2, 1, 3).contiguous() for x in dev[:6]]
    o, s = rwkv_ops_amd.generalized_delta_rule(*dev[:6], initial_state=dev[6], head_first=head_first)
    if head_first:
        o = o.permute(0, 2, 1, 3)
    assert torch.isfinite(o.float()).all() and torch.isfinite(s).all()
    eo, es = rel_l2(o, o_ref), rel_l2(s, s_ref)
    print(f"case {i}: B={B} T={T} H={H} decay={decay} state={state} head_first={head_first}: o={eo:.2e} state={es:.2e}")
    assert eo < TOL and es < TOL, (eo, es)


@pytest.mark.parametrize("i,B,T,H,decay", [(0, 1, 70, 2, "model"), (1, 2, 130, 1, "normal"), (2, 1, 199, 2, "slow"),
                                           (3, 1, 64, 3, "channels"), (4, 2, 33, 2, "mixed")])
def test_random_backward(device, i, B, T, H, decay):
    xs = list(make_inputs(B, T, H, 64, seed=7100 + i, dtype=torch.bfloat16))
    g = torch.Generator().manual_seed(100 + i)
    w = _decays(decay, (B, T, H, 64), g)
    if w is not None:
        xs[1] = w.to(torch.bfloat16)
    dO = torch.randn(B, T, H, 64, generator=g).to(torch.bfloat16)
    dS = 0.1 * torch.randn(B, H, 64, 64, generator=g)
    ref = orc.gradients(*xs[:6], xs[6], dO, dS)
    got = grads_gpu(xs, dO, dS, device)
    for x in got:
        assert torch.isfinite(x.float()).all()
    check(got, ref, f"case {i} ({decay}):")


def _packed_cases():
    rnd = random.Random(20240612)
    out = []
    for i in range(14):
        n_seq = rnd.randint(1, 12)
        lens = [rnd.choice([0, 1, 63, 64, 65]) if rnd.random() < 0.3 else rnd.randint(1, 300) for _ in range(n_seq)]
        if sum(lens) == 0:
            lens[0] = 5
        big = i % 3 == 2                                   # one-kernel form (sequences * heads >= 96, above the threshold of 72)
        H = rnd.randint(96 // n_seq + 1, 128 // n_seq + 8) if big else rnd.randint(1, max(1, 95 // n_seq))
        out.append((i, lens, H, rnd.choice(["model", "normal", "slow", "channels"]), rnd.random() < 0.7,
                    rnd.choice([0, 0, 7])))
    return out


@pytest.mark.parametrize("i,lens,H,decay,with_h0,tail", _packed_cases())
def test_random_packed_forward(device, i, lens, H, decay, with_h0, tail):
    """Packed sequences (cu_seqlens): every sequence against the oracle run on it alone."""
    g = torch.Generator().manual_seed(300 + i)
    T = sum(lens) + tail
    xs = list(make_inputs(1, T, H, 64, seed=7200 + i, dtype=torch.bfloat16, h0=False))
    w = _decays(decay, (1, T, H, 64), g)
    if w is not None:
        xs[1] = w.to(torch.bfloat16)
    h0 = 0.1 * torch.randn(len(lens), H, 64, 64, generator=g) if with_h0 else None
    cu = [0]
    for L in lens:
        cu.append(cu[-1] + L)
    o, s = rwkv_ops_amd.generalized_delta_rule(*[x.to(device) for x in xs[:6]],
                                               initial_state=None if h0 is None else h0.to(device), cu_seqlens=cu)
    assert torch.isfinite(o.float()).all() and torch.isfinite(s).all()
    refs = []
    for j, L in enumerate(lens):
        h0_j = None if h0 is None else h0[j:j + 1]
        if L == 0:
            assert torch.equal(s[j:j + 1].cpu(), h0_j if with_h0 else torch.zeros(1, H, 64, 64))
            continue
        o_ref, s_ref = native_c.run(*[x[:, cu[j]:cu[j + 1]].contiguous() for x in xs[:6]], h0_j)
        refs.append(o_ref)
        assert rel_l2(s[j:j + 1], s_ref) < TOL, (j, L)
    eo = rel_l2(o[:, :cu[-1]], torch.cat(refs, dim=1))
    print(f"case {i}: lens={lens} H={H} decay={decay} h0={with_h0} tail={tail}: o={eo:.2e}")
    assert eo < TOL
    assert torch.count_nonzero(o[:, cu[-1]:]) == 0


def _rwkv6_cases():
    rnd = random.Random(20240613)
    out = []
    for i in range(12):
        big = i % 3 == 2
        B = rnd.randint(1, 4)
        H = rnd.randint(96 // B + 1, 160 // B) if big else rnd.randint(1, max(1, 95 // B))
        T = rnd.choice([1, 2, 63, 64, 65, 129]) if i % 4 == 0 else rnd.randint(1, 260)
        out.append((i, B, T, H, rnd.choice(["normal", "slow", "mixed", "channels"]),
                    rnd.choice(["none", "given", "shared", "mapped"])))
    return out


@pytest.mark.parametrize("i,B,T,H,decay,state", _rwkv6_cases())
def test_random_rwkv6_forward(device, i, B, T, H, decay, state):
    from oracle import rwkv6_native as o6
    g = torch.Generator().manual_seed(400 + i)
    C = H * 64
    r, k, v = (torch.randn(B, T, C, generator=g).to(torch.bfloat16) for _ in range(3))
    w = _decays(decay, (B, T, H, 64), g).reshape(B, T, C).to(torch.bfloat16)
    u = (0.5 * torch.randn(H, 64, generator=g)).to(torch.bfloat16)
    kw = {}
    if state != "none":
        n_state = {"given": B, "shared": 1, "mapped": 3}[state]
        kw["init_state"] = 0.1 * torch.randn(min(n_state, B) if state == "mapped" else n_state, H, 64, 64, generator=g)
        if state == "mapped":
            kw["state_map"] = [rnd_ % kw["init_state"].shape[0] for rnd_ in range(7, 7 + B)]
    y_ref, s_ref = o6.rwkv6(r, k, v, w, u, with_state=True, **kw)
    op = rwkv_ops_amd.RWKV6_OP(64, 4096, state_dtype=torch.float32)
    with torch.no_grad():
        y, s = op(*[x.to(device) for x in (r, k, v, w, u)], with_state=True,
                  **{k_: (v_.to(device) if isinstance(v_, torch.Tensor) else v_) for k_, v_ in kw.items()})
    assert torch.isfinite(y.float()).all() and torch.isfinite(s).all()
    ey, es = rel_l2(y, y_ref), rel_l2(s, s_ref)
    print(f"case {i}: B={B} T={T} H={H} decay={decay} state={state}: y={ey:.2e} state={es:.2e}")
    assert ey < TOL and es < TOL, (ey, es)
