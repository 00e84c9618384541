"""Packed sequences of different lengths (`cu_seqlens`).

The reference declares the argument (torch_op.py:283,338,363-365) and checks it (torch_op.py:388-398) but
never hands it to its kernels, so it holds no values to compare with.  What pins the result is the meaning
the reference documents: sequence i of the packed row is tokens cu_seqlens[i] .. cu_seqlens[i+1]-1 with its
own initial and final state, i.e. the packed call equals one call per sequence.  Checked against the CPU
oracle per sequence (5e-3 relative L2 for bf16, 1e-4 for float32, the tolerances of the dense tests) and,
where both calls take the same kernels, bit for bit against this library's own per-sequence calls.
"""
import pytest
import torch

import rwkv_ops_amd
from oracle import native_c
from oracle import rwkv7_native as orc
from rwkv_ops_amd.synthetic import GRAD_NAMES, GRAD_TOL, make_inputs, rel_l2

pytestmark = pytest.mark.gpu
TOL = 5e-3
GRAD_NAMES = list(GRAD_NAMES)


def pack(lens, H, seed, dtype=torch.bfloat16, tail=0):
    """One packed row [1, sum(lens) + tail, H, 64] per input, the per-sequence pieces, states [N, H, 64, 64]
    and cu_seqlens.  `tail` extra tokens after the last sequence belong to no sequence."""
    parts = [make_inputs(1, max(L, 1), H, 64, seed=seed + i, dtype=dtype) for i, L in enumerate(lens)]
    parts = [[x[:, :L] for x in p[:6]] + [p[6]] for p, L in zip(parts, lens)]
    extra = make_inputs(1, max(tail, 1), H, 64, seed=seed + 999, dtype=dtype)
    packed = [torch.cat([p[j] for p in parts] + ([extra[j][:, :tail]] if tail else []), dim=1).contiguous()
              for j in range(6)]
    h0 = torch.cat([p[6] for p in parts], dim=0).contiguous()
    cu = [0]
    for L in lens:
        cu.append(cu[-1] + L)
    return packed, parts, h0, cu


def check_forward(device, lens, H, seed, with_h0=True, tail=0, cu_on_device=False, dtype=torch.bfloat16, tol=TOL):
    packed, parts, h0, cu = pack(lens, H, seed, dtype, tail)
    cu_arg = torch.tensor(cu, dtype=torch.int64, device=device) if cu_on_device else cu
    o, s = rwkv_ops_amd.generalized_delta_rule(*[x.to(device) for x in packed],
                                               initial_state=h0.to(device) if with_h0 else None,
                                               cu_seqlens=cu_arg)
    torch.cuda.synchronize()
    assert tuple(s.shape) == (len(lens), H, 64, 64) and s.dtype == torch.float32
    worst = 0.0
    refs = []
    for i, (p, L) in enumerate(zip(parts, lens)):
        h0_i = h0[i:i + 1] if with_h0 else None
        if L == 0:                                  # no tokens: the state passes through unchanged
            want = h0_i if with_h0 else torch.zeros(1, H, 64, 64)
            assert torch.equal(s[i:i + 1].cpu(), want), f"sequence {i} (empty)"
            continue
        o_ref, s_ref = native_c.run(*p[:6], h0_i)
        refs.append(o_ref)
        eo, es = rel_l2(o[:, cu[i]:cu[i + 1]], o_ref), rel_l2(s[i:i + 1], s_ref)
        worst = max(worst, eo, es)
        # a relative L2 error estimated from a few hundred values scatters by tens of percent: sequences with
        # fewer than 4096 outputs get twice the tolerance each, and the tolerance itself holds for all together
        assert eo < (tol if L * H * 64 >= 4096 else 2 * tol) and es < tol, (i, L, eo, es)
    assert rel_l2(o[:, :cu[-1]], torch.cat(refs, dim=1)) < tol
    assert torch.count_nonzero(o[:, cu[-1]:]) == 0      # rows that belong to no sequence come back as zeros
    print(f"lens={lens} H={H}: worst rel_l2 {worst:.2e}")
    return o, s, packed, parts, h0, cu


# N*H < 72: summaries + scan (value-split scan); N*H >= 72: the one-kernel form; > 128 sequences*heads in
# the two-kernel form cannot happen through rwkv7_fwd_varlen.  Lengths around the chunk size, a single
# token, empty sequences first / in the middle / last, many short sequences.
@pytest.mark.parametrize("lens,H", [
    ([70, 128, 3, 190], 4),
    ([64], 2), ([1], 1), ([63, 65, 64, 1, 127], 3),
    ([0, 100, 0, 0, 37, 0], 2),
    ([300, 5, 1000, 64, 129], 32),                   # 160 sequence-heads: one-kernel form
    ([0, 200, 0, 77], 40),                           # one-kernel form with empty sequences
    ([17] * 40, 4),                                  # many short sequences
    ([2048, 31], 8),
    ([5, 70] * 150, 1),                              # 300 sequences: the chunk list is built 256 sequences at a time
    ([17000, 100], 1),                               # ... and 256 chunks of a sequence at a time
])
def test_varlen_forward_matches_oracle_per_sequence(device, lens, H):
    check_forward(device, lens, H, seed=7000 + len(lens))


def test_varlen_forward_variants(device):
    check_forward(device, [70, 128, 3, 190], 4, seed=7100, with_h0=False)
    check_forward(device, [70, 128, 3, 190], 48, seed=7101, with_h0=False)
    check_forward(device, [5, 600, 64], 3, seed=7102, cu_on_device=True)
    # tokens after the last sequence belong to no sequence: they do not disturb the sequences
    check_forward(device, [100, 30], 2, seed=7103, tail=50)
    check_forward(device, [100, 30], 64, seed=7104, tail=50)


def test_varlen_forward_float32(device):
    check_forward(device, [70, 128, 3, 0, 190], 2, seed=7200, dtype=torch.float32, tol=1e-4)
    check_forward(device, [70, 30], 2, seed=7201, dtype=torch.float32, tol=1e-4, tail=11)


def test_varlen_equals_separate_calls_bit_for_bit(device):
    """Chunks are counted from each sequence's own first token, so below 72 sequence-heads (both calls
    take the summary + scan kernels) the packed call reproduces the per-sequence calls exactly."""
    lens, H = [70, 128, 30, 190, 64], 4          # (13 tokens or more: shorter dense calls take the recurrent kernel)
    packed, parts, h0, cu = pack(lens, H, seed=7300)
    o, s = rwkv_ops_amd.generalized_delta_rule(*[x.to(device) for x in packed], initial_state=h0.to(device),
                                               cu_seqlens=cu)
    for i, p in enumerate(parts):
        o_i, s_i = rwkv_ops_amd.generalized_delta_rule(*[x.to(device).contiguous() for x in p[:6]],
                                                       initial_state=h0[i:i + 1].to(device))
        assert torch.equal(o[:, cu[i]:cu[i + 1]], o_i), i
        assert torch.equal(s[i:i + 1], s_i), i


def test_varlen_one_sequence_equals_dense_call(device):
    for B_H in (4, 128):
        xs = make_inputs(1, 777, B_H, 64, seed=7400, dtype=torch.bfloat16)
        d = [x.to(device) for x in xs]
        o, s = rwkv_ops_amd.generalized_delta_rule(*d[:6], initial_state=d[6])
        o2, s2 = rwkv_ops_amd.generalized_delta_rule(*d[:6], initial_state=d[6], cu_seqlens=[0, 777])
        assert torch.equal(o, o2) and torch.equal(s, s2)


def grads_packed(packed, h0, cu, dO, dS, device):
    leaves = [x.to(device).requires_grad_(True) for x in packed]
    h = None if h0 is None else h0.to(device).requires_grad_(True)
    o, s = rwkv_ops_amd.generalized_delta_rule(*leaves, initial_state=h, cu_seqlens=cu)
    loss = (o.float() * dO.to(device).float()).sum()
    if dS is not None:
        loss = loss + (s * dS.to(device)).sum()
    return torch.autograd.grad(loss, leaves + ([h] if h is not None else []))


@pytest.mark.parametrize("lens,H", [([70, 128, 3, 190], 2), ([64, 0, 1, 65], 3), ([200, 40], 40)])
def test_varlen_backward_matches_oracle_per_sequence(device, lens, H):
    packed, parts, h0, cu = pack(lens, H, seed=7500 + H, tail=9)
    T = packed[0].shape[1]
    g = torch.Generator().manual_seed(H)
    dO = torch.randn(1, T, H, 64, generator=g).to(torch.bfloat16)
    dS = 0.1 * torch.randn(len(lens), H, 64, 64, generator=g)
    got = grads_packed(packed, h0, cu, dO, dS, device)
    worst = {}
    for i, (p, L) in enumerate(zip(parts, lens)):
        if L == 0:                                   # the state passes through: so does its gradient
            assert torch.equal(got[6][i].cpu(), dS[i]), i
            continue
        ref = orc.gradients(*p[:6], h0[i:i + 1], dO[:, cu[i]:cu[i + 1]], dS[i:i + 1])
        for j, name in enumerate(GRAD_NAMES):
            mine = got[j][i:i + 1] if name == "dh0" else got[j][:, cu[i]:cu[i + 1]]
            e = rel_l2(mine, ref[j])
            worst[name] = max(worst.get(name, 0.0), e)
            assert e < GRAD_TOL[name], (i, L, name, e)
    print(f"lens={lens} H={H}:", " ".join(f"{k}={v:.2e}" for k, v in worst.items()))
    for j in range(6):                               # the nine tokens that belong to no sequence
        assert torch.count_nonzero(got[j][:, cu[-1]:]) == 0


def test_varlen_backward_equals_separate_calls_bit_for_bit(device):
    lens, H = [70, 128, 3, 190, 64], 4
    packed, parts, h0, cu = pack(lens, H, seed=7600)
    g = torch.Generator().manual_seed(1)
    dO = torch.randn(1, cu[-1], H, 64, generator=g).to(torch.bfloat16)
    dS = 0.1 * torch.randn(len(lens), H, 64, 64, generator=g)
    got = grads_packed(packed, h0, cu, dO, dS, device)
    for i, p in enumerate(parts):
        leaves = [x.to(device).contiguous().requires_grad_(True) for x in p[:6]]
        h = h0[i:i + 1].to(device).requires_grad_(True)
        o, s = rwkv_ops_amd.generalized_delta_rule(*leaves, initial_state=h)
        loss = (o.float() * dO[:, cu[i]:cu[i + 1]].to(device).float()).sum() + (s * dS[i:i + 1].to(device)).sum()
        ref = torch.autograd.grad(loss, leaves + [h])
        for j, name in enumerate(GRAD_NAMES):
            mine = got[j][i:i + 1] if name == "dh0" else got[j][:, cu[i]:cu[i + 1]]
            assert torch.equal(mine, ref[j]), (i, name)


def test_varlen_strong_decay_backward(device):
    """Chunks whose decay spans several exponent buckets go through the second backward kernel's list."""
    lens, H = [100, 64, 30], 2
    packed, parts, h0, cu = pack(lens, H, seed=7700)
    g = torch.Generator().manual_seed(2)
    packed[1] = torch.randn(packed[1].shape, generator=g).to(torch.bfloat16)   # w ~ N(0,1): several buckets per chunk
    parts = [[x[:, cu[i]:cu[i + 1]] for x in packed] + [None] for i in range(len(lens))]
    dO = torch.randn(1, cu[-1], H, 64, generator=g).to(torch.bfloat16)
    dS = 0.1 * torch.randn(len(lens), H, 64, 64, generator=g)
    got = grads_packed(packed, h0, cu, dO, dS, device)
    for i, p in enumerate(parts):
        ref = orc.gradients(*p[:6], h0[i:i + 1], dO[:, cu[i]:cu[i + 1]], dS[i:i + 1])
        for j, name in enumerate(GRAD_NAMES):
            mine = got[j][i:i + 1] if name == "dh0" else got[j][:, cu[i]:cu[i + 1]]
            assert torch.isfinite(mine.float()).all()
            e = rel_l2(mine, ref[j])
            assert e < GRAD_TOL[name], (i, name, e)


# float32 rows take the chunked float32 backward over the packed sequences (16-token chunks; its records are laid
# out by (first row / 16) + sequence index): lengths around 16, empty sequences, one sequence per slot, many of them
@pytest.mark.parametrize("lens,H", [([70, 128, 3, 190], 2), ([16, 0, 1, 17, 13, 0, 32], 3), ([200, 40], 40),
                                    ([5] * 70, 1), ([15, 1] * 20, 2)])
def test_varlen_float32_backward_matches_oracle_per_sequence(device, lens, H):
    packed, parts, h0, cu = pack(lens, H, seed=7800 + H, dtype=torch.float32, tail=9)
    T = packed[0].shape[1]
    g = torch.Generator().manual_seed(H)
    dO = torch.randn(1, T, H, 64, generator=g)
    dS = 0.1 * torch.randn(len(lens), H, 64, 64, generator=g)
    got = grads_packed(packed, h0, cu, dO, dS, device)
    worst = 0.0
    for i, (p, L) in enumerate(zip(parts, lens)):
        if L == 0:
            assert torch.equal(got[6][i].cpu(), dS[i]), i
            continue
        ref = orc.gradients(*p[:6], h0[i:i + 1], dO[:, cu[i]:cu[i + 1]], dS[i:i + 1])
        for j, name in enumerate(GRAD_NAMES):
            mine = got[j][i:i + 1] if name == "dh0" else got[j][:, cu[i]:cu[i + 1]]
            assert mine.dtype == torch.float32
            e = rel_l2(mine, ref[j])
            worst = max(worst, e)
            assert e < 1e-4, (i, L, name, e)
    print(f"float32 lens={lens[:8]} H={H}: worst rel_l2 {worst:.2e}")
    for j in range(6):
        assert torch.count_nonzero(got[j][:, cu[-1]:]) == 0


# the second case has more sequence-heads (1200) than the token-by-token kernel has workgroups (1024): some take two
@pytest.mark.parametrize("lens,H,strong_seq", [([100, 64, 0, 30], 2, 1), ([7] * 299 + [20], 4, 299)])
def test_varlen_float32_strong_decay_backward(device, lens, H, strong_seq):
    """One sequence whose decays are too strong for the chunk form: the token-by-token kernel does the whole packed
    call."""
    packed, parts, h0, cu = pack(lens, H, seed=7900, dtype=torch.float32)
    g = torch.Generator().manual_seed(2)
    packed[1] = packed[1].clone()
    packed[1][:, cu[strong_seq]:cu[strong_seq + 1]] = 2.0 + torch.randn(1, lens[strong_seq], H, 64, generator=g)
    parts = [[x[:, cu[i]:cu[i + 1]] for x in packed] + [None] for i in range(len(lens))]
    dO = torch.randn(1, cu[-1], H, 64, generator=g)
    dS = 0.1 * torch.randn(len(lens), H, 64, 64, generator=g)
    got = grads_packed(packed, h0, cu, dO, dS, device)
    for i, (p, L) in enumerate(zip(parts, lens)):
        if L == 0:
            assert torch.equal(got[6][i].cpu(), dS[i]), i
            continue
        ref = orc.gradients(*p[:6], h0[i:i + 1], dO[:, cu[i]:cu[i + 1]], dS[i:i + 1])
        for j, name in enumerate(GRAD_NAMES):
            mine = got[j][i:i + 1] if name == "dh0" else got[j][:, cu[i]:cu[i + 1]]
            assert torch.isfinite(mine).all()
            assert rel_l2(mine, ref[j]) < 1e-4, (i, name)


def test_varlen_bad_table_does_not_fault(device):
    """A table that lies (beyond T, decreasing) gives meaningless values but stays inside the tensors."""
    xs = make_inputs(1, 300, 2, 64, seed=7800, dtype=torch.bfloat16)
    d = [x.to(device) for x in xs[:6]]
    for cu in ([0, 500, 10000], [0, 200, 100, 300], [-5, 100, 300]):
        cu_t = torch.tensor(cu, dtype=torch.int32, device=device)      # device tensors are not read back
        o, s = rwkv_ops_amd.generalized_delta_rule(*d, cu_seqlens=cu_t)
        torch.cuda.synchronize()
        assert tuple(s.shape) == (len(cu) - 1, 2, 64, 64)
    with pytest.raises(ValueError):                                    # a host table is checked
        rwkv_ops_amd.generalized_delta_rule(*d, cu_seqlens=[0, 200, 100, 300])


@pytest.mark.parametrize("H", [4, 40])               # summary + scan kernels; the one-kernel form
def test_varlen_in_a_graph(device, H):
    """Captured with one table, replayed with other lengths in the same device tensor."""
    T = 500
    xs = make_inputs(1, T, H, 64, seed=7900, dtype=torch.bfloat16)
    d = [x.to(device) for x in xs[:6]]
    cu = torch.tensor([0, 100, 350, 500], dtype=torch.int32, device=device)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        rwkv_ops_amd.generalized_delta_rule(*d, cu_seqlens=cu)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o_g, s_g = rwkv_ops_amd.generalized_delta_rule(*d, cu_seqlens=cu)
    for table in ([0, 100, 350, 500], [0, 7, 64, 300], [0, 0, 500, 500]):
        cu.copy_(torch.tensor(table, dtype=torch.int32))
        graph.replay()
        torch.cuda.synchronize()
        o_e, s_e = rwkv_ops_amd.generalized_delta_rule(*d, cu_seqlens=cu.clone())
        last = table[-1]
        assert torch.equal(o_g[:, :last], o_e[:, :last]) and torch.equal(s_g, s_e), table
