"""K = V = 128 (the head size of the reference's own value test, test_script/test_rwkv7_value.py:51): the
decode step, the float32 recurrent forward and the float32 recurrent backward, against the CPU oracle (which is written for any head size).
float32 inputs 1e-4, bf16 inputs 5e-3 relative L2 (the arithmetic is float32 either way; bf16 only rounds o)."""
import pytest
import torch

import rwkv_ops_amd
from oracle import rwkv7_native as orc
from rwkv_ops_amd.synthetic import make_inputs, rel_l2

pytestmark = pytest.mark.gpu
N = 128


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 5e-3)])
@pytest.mark.parametrize("B,T,H", [(1, 1, 1), (2, 37, 3), (1, 130, 2), (3, 1, 5)])
def test_forward_matches_oracle(device, B, T, H, dtype, tol):
    xs = make_inputs(B, T, H, N, seed=9000 + T, dtype=dtype)
    fn, use_kernel = rwkv_ops_amd.get_generalized_delta_rule(128)
    assert use_kernel is True
    with torch.no_grad():
        o, s = fn(*[x.to(device) for x in xs[:6]], initial_state=xs[6].to(device))
    o_ref, s_ref = orc.generalized_delta_rule(*[x.float() for x in xs[:6]], xs[6])
    assert o.dtype == dtype and tuple(s.shape) == (B, H, N, N)
    eo, es = rel_l2(o, o_ref), rel_l2(s, s_ref)
    print(f"B={B} T={T} H={H} {dtype}: rel_l2 o={eo:.2e} state={es:.2e}")
    # bf16 beyond 12 tokens takes the chunked MFMA kernel (bf16 operands: the 5e-3 tolerance holds for the state
    # too); everything else is float32 arithmetic
    assert eo < tol and es < (tol if (dtype == torch.bfloat16 and T > 12) else 1e-4)
    assert rel_l2(s, s_ref.transpose(-1, -2)) > 1e-2


@pytest.mark.parametrize("B,T,H", [(1, 13, 1), (1, 64, 2), (2, 65, 1), (1, 200, 3), (2, 128, 6), (3, 1000, 2), (1, 4096, 4)])
def test_chunked_forward_matches_oracle(device, B, T, H):
    """bf16, K = V = 128, more than 12 tokens: the chunked MFMA kernel for this head size; (2, 128, 6) is the shape
    of the reference's value test (test_script/test_rwkv7_value.py:48-53).  5e-3 relative L2 on o and the state."""
    from oracle import native_c
    xs = make_inputs(B, T, H, N, seed=9300 + T, dtype=torch.bfloat16)
    with torch.no_grad():
        o, s = rwkv_ops_amd.generalized_delta_rule(*[x.to(device) for x in xs[:6]], initial_state=xs[6].to(device))
    o_ref, s_ref = native_c.run(*xs[:6], xs[6])
    eo, es = rel_l2(o, o_ref), rel_l2(s, s_ref)
    print(f"K=128 chunked B={B} T={T} H={H}: rel_l2 o={eo:.2e} state={es:.2e}")
    assert o.dtype == torch.bfloat16 and torch.isfinite(o.float()).all()
    assert eo < 5e-3 and es < 5e-3, (eo, es)
    assert rel_l2(s, s_ref.transpose(-1, -2)) > 1e-2


@pytest.mark.parametrize("wdist", ["normal", "slow", "mixed"])
def test_chunked_forward_decay_ranges(device, wdist):
    """w ~ N(0, 1) (what the reference's smoke test feeds) needs several exponent buckets per chunk."""
    from oracle import native_c
    B, T, H = 2, 256, 2
    xs = list(make_inputs(B, T, H, N, seed=9400, dtype=torch.bfloat16))
    g = torch.Generator().manual_seed(1)
    if wdist == "normal":
        xs[1] = torch.randn(B, T, H, N, generator=g).to(torch.bfloat16)
    elif wdist == "slow":
        xs[1] = (-5.0 + torch.randn(B, T, H, N, generator=g)).to(torch.bfloat16)
    else:
        xs[1] = (3.0 * torch.randn(B, T, H, N, generator=g) - 1.0).to(torch.bfloat16)
    with torch.no_grad():
        o, s = rwkv_ops_amd.generalized_delta_rule(*[x.to(device) for x in xs[:6]], initial_state=xs[6].to(device))
    o_ref, s_ref = native_c.run(*xs[:6], xs[6])
    eo, es = rel_l2(o, o_ref), rel_l2(s, s_ref)
    print(f"K=128 {wdist}: rel_l2 o={eo:.2e} state={es:.2e}")
    assert torch.isfinite(o.float()).all() and torch.isfinite(s).all()
    assert eo < 5e-3 and es < 5e-3, (eo, es)


def test_chunked_forward_variants(device):
    """No initial state, a shared one, a state map, padding by w = -1e9, packed sequences: each against the
    oracle run the plain way."""
    from oracle import native_c
    B, T, H = 3, 150, 2
    xs = make_inputs(B, T, H, N, seed=9500, dtype=torch.bfloat16)
    d = [x.to(device) for x in xs]
    with torch.no_grad():
        o, s = rwkv_ops_amd.generalized_delta_rule(*d[:6])
        o_ref, s_ref = native_c.run(*xs[:6], None)
        assert rel_l2(o, o_ref) < 5e-3 and rel_l2(s, s_ref) < 5e-3
        o, s = rwkv_ops_amd.generalized_delta_rule(*d[:6], initial_state=d[6][:1])
        o_ref, s_ref = native_c.run(*xs[:6], xs[6][:1])
        assert rel_l2(o, o_ref) < 5e-3 and rel_l2(s, s_ref) < 5e-3
        o, s = rwkv_ops_amd.generalized_delta_rule(*d[:6], initial_state=d[6], state_map=[2, 0, 2])
        o_ref, s_ref = native_c.run(*xs[:6], xs[6][[2, 0, 2]])
        assert rel_l2(o, o_ref) < 5e-3 and rel_l2(s, s_ref) < 5e-3
        # the last 40 tokens padded: state untouched by them, outputs zero
        pad = 40
        mask = torch.ones(B, T, 1, 1)
        mask[:, T - pad:] = 0
        ys = [(xs[i].float() * mask).to(torch.bfloat16) if i != 1 else (xs[1].float() + (1 - mask) * -1e9).to(torch.bfloat16)
              for i in range(6)]
        o, s = rwkv_ops_amd.generalized_delta_rule(*[y.to(device) for y in ys], initial_state=d[6])
        o2, s2 = rwkv_ops_amd.generalized_delta_rule(*[y[:, :T - pad].to(device) for y in ys], initial_state=d[6])
        assert torch.equal(s, s2) and torch.equal(o[:, :T - pad], o2) and float(o[:, T - pad:].float().abs().max()) == 0.0
        # packed: lengths 150, 0, 20, 130 in one row of 320 tokens (20 rows behind the last sequence)
        row = [torch.cat([x[0], x[1]], 0)[None].contiguous() for x in d[:6]]          # [1, 300, H, N]
        row = [torch.cat([x, x[:, :20]], 1).contiguous() for x in row]                 # [1, 320, ...]
        cu = [0, 150, 150, 170, 300]
        h4 = torch.cat([d[6], d[6][:1]], 0)
        o, s = rwkv_ops_amd.generalized_delta_rule(*row, initial_state=h4, cu_seqlens=cu)
        for i in range(4):
            a_, b_ = cu[i], cu[i + 1]
            if a_ == b_:
                assert torch.equal(s[i], h4[i])
                continue
            o_ref, s_ref = native_c.run(*[x[:, a_:b_].cpu() for x in row], h4[i:i + 1].cpu())
            tol = 1e-2 if b_ - a_ < 64 else 5e-3
            assert rel_l2(o[:, a_:b_], o_ref) < tol and rel_l2(s[i:i + 1], s_ref) < tol, i
        assert float(o[:, 300:].float().abs().max()) == 0.0


def test_decode_steps_state_pool_and_packed_sequences(device):
    B, T, H = 3, 12, 2
    xs = make_inputs(B, T, H, N, seed=9100, dtype=torch.bfloat16)
    d = [x.to(device) for x in xs]
    o_ref, s_ref = orc.generalized_delta_rule(*[x.float() for x in xs[:6]], xs[6])
    # T single-token steps on a pool of 5 states, rows mapped to slots 4, 0, 2, updated in place
    pool = torch.zeros(5, H, N, N, device=device)
    slots = [4, 0, 2]
    pool[slots] = d[6]
    outs = []
    with torch.no_grad():
        for t in range(T):
            outs.append(rwkv_ops_amd.rwkv7_decode_step(*[x[:, t] for x in d[:6]], pool, state_map=slots))
    assert rel_l2(torch.stack(outs, 1), o_ref) < 5e-3 and rel_l2(pool[slots], s_ref) < 1e-4
    assert torch.count_nonzero(pool[[1, 3]]) == 0
    # the same rows as one packed row with cumulative lengths
    packed = [x.reshape(1, B * T, H, N) for x in d[:6]]
    with torch.no_grad():
        o, s = rwkv_ops_amd.generalized_delta_rule(*packed, initial_state=d[6], cu_seqlens=[0, T, 2 * T, 3 * T])
    # (a packed bf16 row of more than 12 tokens takes the chunked kernel: bf16 operands, 5e-3 on the state too)
    assert rel_l2(o.reshape(B, T, H, N), o_ref) < 5e-3 and rel_l2(s, s_ref) < 5e-3


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 4e-3)])
def test_gradients_at_the_reference_value_test_shape(device, dtype, tol):
    """The shape of the reference's own value test (/root/reference/test_script/test_rwkv7_value.py:48-53:
    T = 128, B = 2, H = 6, head size 128): all seven gradients from the float32 recurrent backward against float32
    autograd through the oracle on the same rounded inputs.  float32: 1e-4; bf16: the gradients are rounded to
    bf16 on store (2^-9 per element), nothing else is."""
    B, T, H = 2, 128, 6
    xs = make_inputs(B, T, H, N, seed=9200, dtype=dtype)
    g = torch.Generator().manual_seed(9201)
    dO = torch.randn(B, T, H, N, generator=g).to(dtype)
    dS = 0.1 * torch.randn(B, H, N, N, generator=g)
    ref = orc.gradients(*xs[:6], xs[6], dO, dS)
    leaves = [x.to(device).requires_grad_(True) for x in xs]
    o, s = rwkv_ops_amd.generalized_delta_rule(*leaves[:6], initial_state=leaves[6])
    loss = (o.float() * dO.to(device).float()).sum() + (s * dS.to(device)).sum()
    got = torch.autograd.grad(loss, leaves)
    errs = {n: rel_l2(g_, r_) for n, g_, r_ in zip(["dr", "dw", "dk", "dv", "da", "db", "dh0"], got, ref)}
    print(f"K=128 {dtype}:", " ".join(f"{k}={v:.2e}" for k, v in errs.items()))
    for name, g_ in zip(errs, got):
        assert g_.dtype == (torch.float32 if name == "dh0" else dtype)
        assert errs[name] < (1e-4 if name == "dh0" else tol), (name, errs)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 4e-3)])
def test_packed_gradients(device, dtype, tol):
    """Packed rows at head size 128: the float32 recurrent backward over the sequences (segments of 32 tokens, their
    records laid out by (first row / 32) + sequence index), each sequence against float32 autograd through the oracle on
    the same rounded inputs; an empty sequence passes its state gradient through; rows behind the last sequence get
    zero gradients."""
    lens, H, tail = [40, 0, 33, 1, 70], 2, 5
    parts = [make_inputs(1, max(L, 1), H, N, seed=9300 + i, dtype=dtype) for i, L in enumerate(lens)]
    parts = [[x[:, :L] for x in p[:6]] + [p[6]] for p, L in zip(parts, lens)]
    extra = make_inputs(1, tail, H, N, seed=9399, dtype=dtype)
    packed = [torch.cat([p[j] for p in parts] + [extra[j]], dim=1).contiguous() for j in range(6)]
    h0 = torch.cat([p[6] for p in parts], dim=0).contiguous()
    cu = [0]
    for L in lens:
        cu.append(cu[-1] + L)
    T = packed[0].shape[1]
    g = torch.Generator().manual_seed(9301)
    dO = torch.randn(1, T, H, N, generator=g).to(dtype)
    dS = 0.1 * torch.randn(len(lens), H, N, N, generator=g)
    leaves = [x.to(device).requires_grad_(True) for x in packed]
    h = h0.to(device).requires_grad_(True)
    o, s = rwkv_ops_amd.generalized_delta_rule(*leaves, initial_state=h, cu_seqlens=cu)
    loss = (o.float() * dO.to(device).float()).sum() + (s * dS.to(device)).sum()
    got = torch.autograd.grad(loss, leaves + [h])
    names = ["dr", "dw", "dk", "dv", "da", "db", "dh0"]
    for i, (p, L) in enumerate(zip(parts, lens)):
        if L == 0:
            assert torch.equal(got[6][i].cpu(), dS[i]), i
            continue
        ref = orc.gradients(*p[:6], h0[i:i + 1], dO[:, cu[i]:cu[i + 1]], dS[i:i + 1])
        for j, name in enumerate(names):
            mine = got[j][i:i + 1] if name == "dh0" else got[j][:, cu[i]:cu[i + 1]]
            e = rel_l2(mine, ref[j])
            # (a relative L2 error over a few hundred values scatters: short sequences get twice the tolerance)
            assert e < (1e-4 if name == "dh0" else (tol if L * H * N >= 4096 else 2 * tol)), (i, L, name, e)
    for j in range(6):
        assert got[j].dtype == dtype and torch.count_nonzero(got[j][:, cu[-1]:]) == 0


@pytest.mark.parametrize("T", [20, 7, 37])
def test_gradients_with_many_heads(device, T):
    """At most 192 (batch, head) pairs: the value columns of a head are split over two workgroups, whose partial sums
    a second kernel adds (the shapes above); beyond: one workgroup per pair.  Here 208 pairs, and the same tensors'
    first 3 batch rows (24 pairs) through the split form: both against float32 autograd through the oracle, and
    against each other (different orders of the same float32 sums)."""
    B, H = 26, 8
    xs = make_inputs(B, T, H, N, seed=9500, dtype=torch.float32)
    g = torch.Generator().manual_seed(9501)
    dO = torch.randn(B, T, H, N, generator=g)
    dS = 0.1 * torch.randn(B, H, N, N, generator=g)
    ref = orc.gradients(*xs[:6], xs[6], dO, dS)
    got = {}
    for rows in (B, 3):
        leaves = [x[:rows].contiguous().to(device).requires_grad_(True) for x in xs]
        o, s = rwkv_ops_amd.generalized_delta_rule(*leaves[:6], initial_state=leaves[6])
        loss = (o * dO[:rows].to(device)).sum() + (s * dS[:rows].to(device)).sum()
        got[rows] = torch.autograd.grad(loss, leaves)
        for name, g_, r_ in zip(["dr", "dw", "dk", "dv", "da", "db", "dh0"], got[rows], ref):
            assert rel_l2(g_, r_[:rows]) < 1e-4, (rows, name)
    for a_, b_ in zip(got[B], got[3]):
        assert rel_l2(a_[:3], b_) < 2e-6


def test_gradients_at_the_benchmark_shape(device):
    """B = 8, T = 1024, H = 16, bf16 (bench.py's head128.backward: 128 (batch, head) pairs, so the split form on all
    256 CUs): four pairs, the corners of the batch among them, against float32 autograd through the oracle on the
    same rounded inputs (heads and batch rows are independent, so the oracle runs on the slices)."""
    B, T, H = 8, 1024, 16
    xs = make_inputs(B, T, H, N, seed=9600, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(9601)
    dO = torch.randn(B, T, H, N, generator=g).to(torch.bfloat16)
    dS = 0.1 * torch.randn(B, H, N, N, generator=g)
    leaves = [x.to(device).requires_grad_(True) for x in xs]
    o, s = rwkv_ops_amd.generalized_delta_rule(*leaves[:6], initial_state=leaves[6])
    loss = (o.float() * dO.to(device).float()).sum() + (s * dS.to(device)).sum()
    got = [t.cpu() for t in torch.autograd.grad(loss, leaves)]
    names = ["dr", "dw", "dk", "dv", "da", "db", "dh0"]
    for b, h in ((0, 0), (B - 1, H - 1), (0, H - 1), (3, 7)):
        one = [x[b:b + 1, :, h:h + 1].contiguous() for x in xs[:6]] + [xs[6][b:b + 1, h:h + 1].contiguous()]
        ref = orc.gradients(*one[:6], one[6], dO[b:b + 1, :, h:h + 1].contiguous(), dS[b:b + 1, h:h + 1].contiguous())
        for j, name in enumerate(names):
            mine = got[j][b:b + 1, h:h + 1] if name == "dh0" else got[j][b:b + 1, :, h:h + 1]
            e = rel_l2(mine, ref[j])
            assert e < (1e-4 if name == "dh0" else 4e-3), (b, h, name, e)


@pytest.mark.parametrize("B,H", [(3, 2), (50, 4)])
def test_float32_forward_variants(device, B, H):
    """float32 tensors at head size 128 take the recurrent forward: two workgroups per (batch, head) up to 192 pairs
    (6 here), one beyond (200).  No initial state, a shared one, a state map, packed sequences with an empty one and
    rows behind the last: against the oracle, 1e-4."""
    from oracle import native_c
    T = 45
    xs = make_inputs(B, T, H, N, seed=9700, dtype=torch.float32)
    d = [x.to(device) for x in xs]
    with torch.no_grad():
        o, s = rwkv_ops_amd.generalized_delta_rule(*d[:6])
        o_ref, s_ref = native_c.run(*xs[:6], None)
        assert rel_l2(o, o_ref) < 1e-4 and rel_l2(s, s_ref) < 1e-4
        o, s = rwkv_ops_amd.generalized_delta_rule(*d[:6], initial_state=d[6][:1])
        o_ref, s_ref = native_c.run(*xs[:6], xs[6][:1])
        assert rel_l2(o, o_ref) < 1e-4 and rel_l2(s, s_ref) < 1e-4
        smap = [(2 * i + 1) % B for i in range(B)]
        o, s = rwkv_ops_amd.generalized_delta_rule(*d[:6], initial_state=d[6], state_map=smap)
        o_ref, s_ref = native_c.run(*xs[:6], xs[6][smap])
        assert rel_l2(o, o_ref) < 1e-4 and rel_l2(s, s_ref) < 1e-4
        # the first two batch rows as one packed row: lengths 45, 0, 30, 15, and 10 rows behind the last sequence
        row = [torch.cat([x[0], x[1], x[2][:10]], 0)[None].contiguous() for x in d[:6]]
        cu = [0, 45, 45, 75, 90]
        h4 = d[6][[0, 1, 2, 0]].contiguous()
        o, s = rwkv_ops_amd.generalized_delta_rule(*row, initial_state=h4, cu_seqlens=cu)
        for i in range(4):
            a_, b_ = cu[i], cu[i + 1]
            if a_ == b_:
                assert torch.equal(s[i], h4[i])
                continue
            o_ref, s_ref = native_c.run(*[x[:, a_:b_].cpu() for x in row], h4[i:i + 1].cpu())
            assert rel_l2(o[:, a_:b_], o_ref) < 1e-4 and rel_l2(s[i:i + 1], s_ref) < 1e-4, i
        assert float(o[:, 90:].abs().max()) == 0.0
