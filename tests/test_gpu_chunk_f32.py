"""The chunked float32 forward (float32 tensors, K = V = 64, more than 12 tokens: 16-token chunks on the float32
matrix cores) against the CPU oracle, the restatement of the reference's native loop
(/root/reference/rwkv_ops/rwkv7_kernel/native_keras_op.py:80-88).  Tolerance: the task's float32 tolerance, 1e-4
relative L2 on o and the final state (measured: a few 1e-7); and 1e-5 against this library's own token-by-token
float32 kernel, the two being different orders of the same float32 arithmetic."""
import ctypes

import pytest
import torch

import rwkv_ops_amd
from oracle import native_c
from rwkv_ops_amd.rwkv7 import _lib
from rwkv_ops_amd.synthetic import make_inputs, rel_l2

pytestmark = pytest.mark.gpu
N = 64
TOL = 1e-4


def recurrent(d, h0):
    """the token-by-token float32 kernel through the C ABI"""
    lib = _lib.load()
    B, T, H, _ = d[0].shape
    o, s = torch.empty_like(d[0]), torch.empty(B, H, N, N, device=d[0].device)
    rc = lib.rwkv7_fwd_recurrent(*[x.data_ptr() for x in d[:6]], h0.data_ptr() if h0 is not None else None,
                                 H * N * N, o.data_ptr(), s.data_ptr(), B, T, H, N, N, _lib.DTYPE_F32,
                                 torch.cuda.current_stream().cuda_stream)
    assert rc == 0, rc
    return o, s


@pytest.mark.parametrize("B,T,H", [(1, 13, 1), (2, 16, 3), (1, 17, 2), (3, 31, 1), (2, 32, 2), (1, 33, 5),
                                   (2, 100, 3), (1, 257, 4), (2, 1000, 2)])
def test_matches_oracle(device, B, T, H):
    xs = make_inputs(B, T, H, N, seed=9600 + T, dtype=torch.float32)
    with torch.no_grad():
        o, s = rwkv_ops_amd.generalized_delta_rule(*[x.to(device) for x in xs[:6]], initial_state=xs[6].to(device))
    o_ref, s_ref = native_c.run(*xs[:6], xs[6])
    eo, es = rel_l2(o, o_ref), rel_l2(s, s_ref)
    print(f"float32 chunked B={B} T={T} H={H}: rel_l2 o={eo:.2e} state={es:.2e}")
    assert o.dtype == torch.float32 and torch.isfinite(o).all()
    assert eo < TOL and es < 1e-5, (eo, es)
    assert rel_l2(s, s_ref.transpose(-1, -2)) > 1e-2


@pytest.mark.parametrize("wdist", ["normal", "strong", "slow", "some_channels", "one_chunk_in_three"])
def test_decay_ranges(device, wdist):
    """A chunk whose decay is too strong for k e^{-gi} is walked token by token, by all waves together, whichever
    wave's channels it is that decay; chunks of both kinds follow one another in a sequence."""
    B, T, H = 2, 150, 2
    xs = list(make_inputs(B, T, H, N, seed=9700, dtype=torch.float32))
    g = torch.Generator().manual_seed(2)
    if wdist == "normal":
        xs[1] = torch.randn(B, T, H, N, generator=g)                  # what the reference's smoke test feeds
    elif wdist == "strong":
        xs[1] = 2.0 + torch.randn(B, T, H, N, generator=g)
    elif wdist == "slow":
        xs[1] = -6.0 + torch.randn(B, T, H, N, generator=g)
    elif wdist == "some_channels":
        xs[1] = xs[1].clone()
        xs[1][..., 37] = 3.0                                           # one channel (third wave's) decays by e^-20 a step
    else:
        xs[1] = xs[1].clone()
        for c in range(0, T // 16, 3):
            xs[1][:, 16 * c:16 * c + 16] = 2.5
    with torch.no_grad():
        o, s = rwkv_ops_amd.generalized_delta_rule(*[x.to(device) for x in xs[:6]], initial_state=xs[6].to(device))
    o_ref, s_ref = native_c.run(*xs[:6], xs[6])
    eo, es = rel_l2(o, o_ref), rel_l2(s, s_ref)
    print(f"float32 chunked {wdist}: rel_l2 o={eo:.2e} state={es:.2e}")
    assert torch.isfinite(o).all() and torch.isfinite(s).all()
    assert eo < TOL and es < TOL, (eo, es)


@pytest.mark.parametrize("B,T,H", [(4, 2048, 8), (1, 4097, 3), (40, 64, 16)])
def test_matches_the_recurrent_kernel(device, B, T, H):
    xs = make_inputs(B, T, H, N, seed=9800, dtype=torch.float32)
    d = [x.to(device) for x in xs]
    with torch.no_grad():
        o, s = rwkv_ops_amd.generalized_delta_rule(*d[:6], initial_state=d[6])
    o2, s2 = recurrent(d, d[6])
    eo, es = rel_l2(o, o2), rel_l2(s, s2)
    print(f"float32 chunked vs recurrent B={B} T={T} H={H}: o={eo:.2e} state={es:.2e}")
    assert eo < 1e-5 and es < 1e-5, (eo, es)


def test_variants(device):
    """No initial state, a shared one, a state map, padding by w = -1e9 (a strong chunk), packed sequences with an
    empty one and rows behind the last: each against the oracle run the plain way."""
    B, T, H = 3, 150, 2
    xs = make_inputs(B, T, H, N, seed=9900, dtype=torch.float32)
    d = [x.to(device) for x in xs]
    with torch.no_grad():
        o, s = rwkv_ops_amd.generalized_delta_rule(*d[:6])
        o_ref, s_ref = native_c.run(*xs[:6], None)
        assert rel_l2(o, o_ref) < TOL and rel_l2(s, s_ref) < 1e-5
        o, s = rwkv_ops_amd.generalized_delta_rule(*d[:6], initial_state=d[6][:1])
        o_ref, s_ref = native_c.run(*xs[:6], xs[6][:1])
        assert rel_l2(o, o_ref) < TOL and rel_l2(s, s_ref) < 1e-5
        o, s = rwkv_ops_amd.generalized_delta_rule(*d[:6], initial_state=d[6], state_map=[2, 0, 2])
        o_ref, s_ref = native_c.run(*xs[:6], xs[6][[2, 0, 2]])
        assert rel_l2(o, o_ref) < TOL and rel_l2(s, s_ref) < 1e-5
        # the last 40 tokens padded: state untouched by them, outputs zero
        pad = 40
        mask = torch.ones(B, T, 1, 1)
        mask[:, T - pad:] = 0
        ys = [xs[i] * mask if i != 1 else xs[1] + (1 - mask) * -1e9 for i in range(6)]
        o, s = rwkv_ops_amd.generalized_delta_rule(*[y.to(device) for y in ys], initial_state=d[6])
        o2, s2 = rwkv_ops_amd.generalized_delta_rule(*[y[:, :T - pad].contiguous().to(device) for y in ys], initial_state=d[6])
        assert rel_l2(s, s2) < 1e-6 and rel_l2(o[:, :T - pad], o2) < 1e-6 and float(o[:, T - pad:].abs().max()) == 0.0
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
            assert rel_l2(o[:, a_:b_], o_ref) < TOL and rel_l2(s[i:i + 1], s_ref) < 1e-5, i
        assert float(o[:, 300:].abs().max()) == 0.0
        # packed, without an initial state: the empty sequence's final state is zero
        o, s = rwkv_ops_amd.generalized_delta_rule(*row, cu_seqlens=cu)
        assert float(s[1].abs().max()) == 0.0


def test_through_the_c_abi_without_a_workspace(device):
    """rwkv7_fwd on float32 tensors takes no workspace (NULL, 0), like the token-by-token kernel it replaces here."""
    lib = _lib.load()
    B, T, H = 2, 77, 3
    xs = make_inputs(B, T, H, N, seed=9950, dtype=torch.float32)
    d = [x.to(device) for x in xs]
    o, s = torch.empty_like(d[0]), torch.empty_like(d[6])
    assert lib.rwkv7_fwd_workspace_bytes(B, T, H, _lib.DTYPE_F32) == 0
    rc = lib.rwkv7_fwd(*[x.data_ptr() for x in d[:6]], d[6].data_ptr(), H * N * N, o.data_ptr(), s.data_ptr(),
                       B, T, H, N, N, _lib.DTYPE_F32, None, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    o_ref, s_ref = native_c.run(*xs[:6], xs[6])
    assert rel_l2(o, o_ref) < TOL and rel_l2(s, s_ref) < 1e-5
