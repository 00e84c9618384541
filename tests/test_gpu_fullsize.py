"""GPU parity at the benchmark configurations' full sizes.

Forward results are compared with the C restatement of the reference's native loop
(oracle/rwkv7_native.c, float32, OpenMP) on the same seeded bf16-rounded inputs; gradients with
torch autograd through the oracle on a slice of (batch, head) sequences, which are independent of
one another.  Tolerances: 1e-4 (float32 inputs) and 5e-3 (bf16 inputs) relative L2 on o and the final
state, as the task states; gradients as in tests/test_gpu_backward.py.
"""
import pytest
import torch

import rwkv_ops_amd
from oracle import native_c
from oracle import rwkv7_native as orc
from rwkv_ops_amd.synthetic import GRAD_TOL, make_inputs, rel_l2

pytestmark = pytest.mark.gpu


def test_config0_float32_native_shape(device):
    # B=1, T=256, H=4, float32, head_first=False, initial state in, final state out
    xs = make_inputs(1, 256, 4, 64, seed=1234, dtype=torch.float32)
    o_ref, s_ref = orc.generalized_delta_rule(*xs[:6], xs[6])
    o, s = rwkv_ops_amd.generalized_delta_rule(*[x.to(device) for x in xs])
    assert o.dtype == torch.float32 and s.dtype == torch.float32
    eo, es = rel_l2(o, o_ref), rel_l2(s, s_ref)
    print(f"config 0: rel_l2 o={eo:.2e} state={es:.2e}")
    assert eo < 1e-4 and es < 1e-4


def test_config1_prefill_full_size(device):
    B, T, H = 8, 4096, 32
    xs = make_inputs(B, T, H, 64, seed=1235, dtype=torch.bfloat16)
    o_ref, s_ref = native_c.run(*xs[:6], xs[6])
    o, s = rwkv_ops_amd.generalized_delta_rule(*[x.to(device) for x in xs])
    eo, es = rel_l2(o, o_ref), rel_l2(s, s_ref)
    print(f"config 1: rel_l2 o={eo:.2e} state={es:.2e}")
    assert eo < 5e-3 and es < 5e-3
    # per-(batch, head) worst case
    num = (o.float().cpu() - o_ref).pow(2).sum(dim=(1, 3)).sqrt()
    den = o_ref.pow(2).sum(dim=(1, 3)).sqrt()
    assert float((num / den).max()) < 5e-3


def test_config2_decode_full_size(device):
    B, H, steps = 256, 40, 64
    xs = make_inputs(B, steps, H, 64, seed=1236, dtype=torch.bfloat16)
    o_ref, s_ref = native_c.run(*xs[:6], xs[6])
    r, w, k, v, a, b, h0 = [x.to(device) for x in xs]
    state = h0.clone()
    outs = []
    for t in range(steps):
        outs.append(rwkv_ops_amd.rwkv7_decode_step(r[:, t], w[:, t], k[:, t], v[:, t], a[:, t], b[:, t], state))
    o = torch.stack(outs, 1)
    eo, es = rel_l2(o, o_ref), rel_l2(state, s_ref)
    print(f"config 2: rel_l2 o={eo:.2e} state={es:.2e}")
    assert eo < 5e-3 and es < 5e-3
    # the T=1 path of the operator API gives the same numbers as the in-place step
    o1, s1 = rwkv_ops_amd.generalized_delta_rule(r[:, :1], w[:, :1], k[:, :1], v[:, :1], a[:, :1], b[:, :1], h0)
    assert torch.equal(o1[:, 0], outs[0])


def test_config3_long_context_with_padding(device):
    B, T, H, pad = 1, 16384, 64, 1024
    xs = list(make_inputs(B, T, H, 64, seed=1237, dtype=torch.bfloat16, h0=False))
    mask = torch.ones(B, T, 1, 1)
    mask[:, T - pad:] = 0
    for i in (0, 2, 3, 4, 5):
        xs[i] = (xs[i].float() * mask).to(torch.bfloat16)
    xs[1] = (xs[1].float() + (1 - mask) * -1e9).to(torch.bfloat16)      # w += (1-mask)*-1e9
    o_ref, s_ref = native_c.run(*xs[:6], None)
    dev = [x.to(device) for x in xs[:6]]
    o, s = rwkv_ops_amd.generalized_delta_rule(*dev, initial_state=None)
    eo, es = rel_l2(o, o_ref), rel_l2(s, s_ref)
    print(f"config 3: rel_l2 o={eo:.2e} state={es:.2e}")
    assert eo < 5e-3 and es < 5e-3
    # the masked tail leaves the state bitwise untouched and outputs exactly zero
    o2, s2 = rwkv_ops_amd.generalized_delta_rule(*[x[:, :T - pad] for x in dev], initial_state=None)
    assert torch.equal(s2, s) and torch.equal(o2, o[:, :T - pad])
    assert float(o[:, T - pad:].float().abs().max()) == 0.0


def test_config4_forward_backward_full_size(device):
    B, T, H = 4, 2048, 32
    xs = make_inputs(B, T, H, 64, seed=1238, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(4)
    dO = torch.randn(B, T, H, 64, generator=g).to(torch.bfloat16)
    dS = 0.1 * torch.randn(B, H, 64, 64, generator=g)
    leaves = [x.to(device).requires_grad_(True) for x in xs[:6]]
    h0 = xs[6].to(device).requires_grad_(True)
    o, s = rwkv_ops_amd.generalized_delta_rule(*leaves, initial_state=h0)
    loss = (o.float() * dO.to(device).float()).sum() + (s * dS.to(device)).sum()
    got = torch.autograd.grad(loss, leaves + [h0])
    o_ref, s_ref = native_c.run(*xs[:6], xs[6])
    assert rel_l2(o, o_ref) < 5e-3 and rel_l2(s, s_ref) < 5e-3
    # gradients on eight independent (batch, head) sequences, the corners of the batch among them, run through
    # the oracle as one batch of one-head sequences
    pairs = [(0, 0), (0, H - 1), (B - 1, 0), (B - 1, H - 1), (1, 5), (1, 6), (2, 17), (3, 12)]
    bi = torch.tensor([p[0] for p in pairs])
    hi = torch.tensor([p[1] for p in pairs])
    pick = lambda x: x[bi, :, hi].unsqueeze(2)                 # [8, T, 1, 64]
    pick_s = lambda x: x[bi, hi].unsqueeze(1)                  # [8, 1, 64, 64]
    ref = orc.gradients(*[pick(x) for x in xs[:6]], pick_s(xs[6]), pick(dO), pick_s(dS))
    names = ["dr", "dw", "dk", "dv", "da", "db", "dh0"]
    tol = GRAD_TOL
    errs = {}
    for name, gg, rr in zip(names[:6], got[:6], ref[:6]):
        errs[name] = rel_l2(pick(gg.cpu()), rr)
    errs["dh0"] = rel_l2(pick_s(got[6].cpu()), ref[6])
    print("config 4:", " ".join(f"{k}={v:.2e}" for k, v in errs.items()))
    for k_, v_ in errs.items():
        assert v_ < tol[k_], (k_, v_)
    # and each of the eight on its own, so that no single sequence hides behind the others
    for j, pr in enumerate(pairs):
        for name, gg, rr in zip(names[:6], got[:6], ref[:6]):
            e = rel_l2(pick(gg.cpu())[j], rr[j])
            assert e < 1.2 * tol[name], (pr, name, e)
    for gg in got:
        assert torch.isfinite(gg.float()).all()


def _inputs_on_device(B, T, H, device, seed):
    """The benchmark distributions generated on the GPU (a multi-gigabyte case is too slow to draw on the host)."""
    g = torch.Generator(device=device).manual_seed(seed)
    shp = (B, T, H, 64)
    rn = lambda: torch.randn(shp, generator=g, device=device)
    r, k, v = rn().bfloat16(), rn().bfloat16(), rn().bfloat16()
    w = (-torch.exp(-torch.nn.functional.softplus(-rn()) - 0.5)).bfloat16()
    kk = torch.nn.functional.normalize(rn(), dim=-1)
    a = (-kk).bfloat16()
    b = (kk * torch.sigmoid(rn())).bfloat16()
    h0 = 0.1 * torch.randn((B, H, 64, 64), generator=g, device=device)
    return r, w, k, v, a, b, h0


def test_offsets_beyond_32_bits(device):
    """Maximum sizes: 2.7 G elements (5.4 GB) per tensor, so the last batch row lies past both the 4 GiB byte
    offset and the 2^31 element index that 32-bit arithmetic would wrap at.  Sequences are independent, so
    that row computed alone (same kernels, small addresses) must give the same bits, forward and backward."""
    B, T, H = 16, 16384, 160
    free, _ = torch.cuda.mem_get_info()
    if free < 200 * 2**30:
        pytest.skip("needs about 170 GB of device memory")
    xs = _inputs_on_device(B, T, H, device, seed=77)
    o, s = rwkv_ops_amd.generalized_delta_rule(*xs[:6], initial_state=xs[6])
    last = [x[B - 1:].contiguous() for x in xs]
    o1, s1 = rwkv_ops_amd.generalized_delta_rule(*last[:6], initial_state=last[6])
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all() and torch.equal(o[B - 1:], o1) and torch.equal(s[B - 1:], s1)
    del o, o1

    from rwkv_ops_amd.rwkv7.op import rwkv7_bwd
    g = torch.Generator(device=device).manual_seed(78)
    d_o = torch.randn((B, T, H, 64), generator=g, device=device).bfloat16()
    d_s = 0.1 * torch.randn((B, H, 64, 64), generator=g, device=device)
    grads = rwkv7_bwd(*xs[:6], xs[6], d_o, d_s)
    grads1 = rwkv7_bwd(*last[:6], last[6], d_o[B - 1:].contiguous(), d_s[B - 1:].contiguous())
    torch.cuda.synchronize()
    for full, alone in zip(grads, grads1):
        assert torch.equal(full[B - 1:], alone)
