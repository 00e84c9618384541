"""The chunked float32 backward (rwkv7_bwd on float32 tensors, K = V = 64, more than 12 tokens: 16-token chunks on
the float32 matrix cores) against float32 autograd through the CPU oracle, the restatement of the reference's
native loop (/root/reference/rwkv_ops/rwkv7_kernel/native_keras_op.py:80-88).  Tolerance: the task's float32
tolerance, 1e-4 relative L2 on each of the seven gradients (measured: below 1e-6); and 1e-5 against this library's
own token-by-token float32 backward, the two being different orders of the same float32 arithmetic."""
import pytest
import torch

import rwkv_ops_amd
from oracle import rwkv7_native as orc
from rwkv_ops_amd.rwkv7 import _lib
from rwkv_ops_amd.synthetic import GRAD_NAMES, make_inputs, rel_l2

pytestmark = pytest.mark.gpu
N = 64
TOL = 1e-4


def run(device, xs, dO, dS, entry="rwkv7_bwd", ws_bytes=None):
    """the seven gradients through the C ABI; outputs start as NaN so that anything left unwritten shows"""
    lib = _lib.load()
    B, T, H, _ = xs[0].shape
    dev = [x.to(device) for x in xs[:6]]
    h0 = None if xs[6] is None else xs[6].to(device)
    dO_d = None if dO is None else dO.to(device)
    dS_d = None if dS is None else dS.to(device)
    grads = [torch.full_like(dev[0], float("nan")) for _ in range(6)]
    dh0 = torch.full((B, H, N, N), float("nan"), device=device)
    size = (lib.rwkv7_bwd_workspace_bytes(B, T, H, _lib.DTYPE_F32) if entry == "rwkv7_bwd"
            else lib.rwkv7_bwd_recurrent_workspace_bytes(B, T, H, N))
    if ws_bytes is not None:
        size = ws_bytes
    ws = torch.empty(max(size, 1), dtype=torch.uint8, device=device)
    p = lambda t: None if t is None else t.data_ptr()
    h0_stride = 0 if h0 is None or h0.shape[0] == 1 else H * N * N
    rc = getattr(lib, entry)(*[p(x) for x in dev], p(h0), h0_stride, p(dO_d), p(dS_d), *[p(g) for g in grads], p(dh0),
                             B, T, H, N, N, _lib.DTYPE_F32, p(ws), size, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return rc, grads + [dh0]


def upstream(B, T, H, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(B, T, H, N, generator=g), 0.1 * torch.randn(B, H, N, N, generator=g)


@pytest.mark.parametrize("B,T,H", [(1, 13, 1), (2, 16, 3), (1, 17, 2), (3, 31, 1), (2, 32, 2), (1, 33, 5), (2, 100, 3),
                                   (1, 257, 4), (2, 600, 2)])
def test_matches_oracle_autograd(device, B, T, H):
    xs = make_inputs(B, T, H, N, seed=9100 + T, dtype=torch.float32)
    dO, dS = upstream(B, T, H, T)
    ref = orc.gradients(*xs[:6], xs[6], dO, dS)
    rc, got = run(device, xs, dO, dS)
    assert rc == 0, rc
    errs = {n: rel_l2(a_, b_) for n, a_, b_ in zip(GRAD_NAMES, got, ref)}
    print(f"float32 chunked backward B={B} T={T} H={H}:", " ".join(f"{k}={v:.2e}" for k, v in errs.items()))
    for n in GRAD_NAMES:
        assert errs[n] < TOL, (n, errs)


# (4, 2048, 32) is the training shape of the benchmark (BASELINE config 4) in float32
@pytest.mark.parametrize("B,T,H", [(4, 1024, 8), (1, 2049, 3), (40, 64, 4), (4, 2048, 32)])
def test_matches_the_recurrent_backward(device, B, T, H):
    xs = make_inputs(B, T, H, N, seed=9200, dtype=torch.float32)
    dO, dS = upstream(B, T, H, 5)
    rc, got = run(device, xs, dO, dS)
    rc2, ref = run(device, xs, dO, dS, entry="rwkv7_bwd_recurrent")
    assert rc == 0 and rc2 == 0
    errs = {n: rel_l2(a_, b_) for n, a_, b_ in zip(GRAD_NAMES, got, ref)}
    print(f"float32 chunked vs recurrent backward B={B} T={T} H={H}:", " ".join(f"{k}={v:.2e}" for k, v in errs.items()))
    for n in GRAD_NAMES:
        assert errs[n] < 1e-5, (n, errs)


def test_variants(device):
    """No gradient into the final state, none into the outputs, no initial state, one initial state for the whole
    batch; a tail padded by the w = -1e9 convention."""
    B, T, H = 2, 90, 2
    xs = list(make_inputs(B, T, H, N, seed=9300, dtype=torch.float32))
    dO, dS = upstream(B, T, H, 3)
    for d_o, d_s, h0 in ((dO, None, xs[6]), (None, dS, xs[6]), (dO, dS, None), (dO, dS, xs[6][:1].contiguous())):
        ys = xs[:6] + [h0]
        ref = orc.gradients(*ys[:6], h0, d_o, d_s)
        rc, got = run(device, ys, d_o, d_s)
        assert rc == 0
        for n, a_, b_ in zip(GRAD_NAMES[:6], got, ref):
            assert rel_l2(a_, b_) < TOL, (n, d_o is None, d_s is None, h0 is None)
        if h0 is not None:
            # dh0 comes per batch entry; the oracle sums over the batch when the state is shared
            mine = got[6] if h0.shape[0] == B else got[6].sum(0, keepdim=True)
            assert rel_l2(mine, ref[6]) < TOL
    pad = 20
    mask = torch.ones(B, T, 1, 1)
    mask[:, T - pad:] = 0
    ys = [xs[i] * mask if i != 1 else xs[1] + (1 - mask) * -1e9 for i in range(6)] + [xs[6]]
    rc, got = run(device, ys, dO * mask, dS)
    zs = [y[:, :T - pad].contiguous() for y in ys[:6]] + [xs[6]]
    ref = orc.gradients(*zs[:6], xs[6], dO[:, :T - pad].contiguous(), dS)
    for n, a_, b_ in zip(GRAD_NAMES[:6], got, ref):
        assert rel_l2(a_[:, :T - pad], b_) < TOL, n
        assert float(a_[:, T - pad:].abs().max()) == 0.0, n
    assert rel_l2(got[6], ref[6]) < TOL


def test_many_heads_and_no_upstream_gradient(device):
    """More (batch, head) pairs than a workgroup has threads (the flags are read in a loop), with a strong chunk in the
    last one only; and a call with neither upstream gradient, whose seven results are zero."""
    B, T, H = 25, 20, 40
    xs = list(make_inputs(B, T, H, N, seed=9700, dtype=torch.float32))
    dO, dS = upstream(B, T, H, 8)
    rc, got = run(device, xs, dO, dS)
    rc2, ref = run(device, xs, dO, dS, entry="rwkv7_bwd_recurrent")
    assert rc == 0 and rc2 == 0
    for n, a_, b_ in zip(GRAD_NAMES, got, ref):
        assert rel_l2(a_, b_) < 1e-5 and not torch.equal(a_, b_), n      # the chunk form ran
    xs[1] = xs[1].clone()
    xs[1][B - 1, :16, H - 1] = 2.5
    rc, got = run(device, xs, dO, dS)
    rc2, ref = run(device, xs, dO, dS, entry="rwkv7_bwd_recurrent")
    for n, a_, b_ in zip(GRAD_NAMES, got, ref):
        assert torch.equal(a_, b_), n                                    # the token-by-token kernel ran
    rc, got = run(device, list(make_inputs(2, 50, 2, N, seed=9701, dtype=torch.float32)), None, None)
    assert rc == 0
    for n, a_ in zip(GRAD_NAMES, got):
        assert float(a_.abs().max()) == 0.0, n


@pytest.mark.parametrize("wdist", ["normal", "strong", "one_chunk"])
def test_strong_decays_take_the_token_by_token_kernel(device, wdist):
    """A chunk whose decay is too strong for k e^{-gi} anywhere in the call: the whole call is done by the
    token-by-token kernel, bit for bit what rwkv7_bwd_recurrent returns."""
    B, T, H = 2, 150, 2
    xs = list(make_inputs(B, T, H, N, seed=9400, dtype=torch.float32))
    g = torch.Generator().manual_seed(2)
    if wdist == "normal":
        xs[1] = torch.randn(B, T, H, N, generator=g)                  # what the reference's smoke test feeds
    elif wdist == "strong":
        xs[1] = 2.0 + torch.randn(B, T, H, N, generator=g)
    else:
        xs[1] = xs[1].clone()
        xs[1][1, 32:48, 1] = 2.5                                       # one chunk of one head
    dO, dS = upstream(B, T, H, 4)
    rc, got = run(device, xs, dO, dS)
    rc2, ref = run(device, xs, dO, dS, entry="rwkv7_bwd_recurrent")
    assert rc == 0 and rc2 == 0
    for n, a_, b_ in zip(GRAD_NAMES, got, ref):
        assert torch.isfinite(a_).all(), n
        if wdist != "normal":
            assert torch.equal(a_, b_), n
        else:
            assert rel_l2(a_, b_) < 1e-5, n
    want = orc.gradients(*xs[:6], xs[6], dO, dS)
    for n, a_, b_ in zip(GRAD_NAMES, got, want):
        assert rel_l2(a_, b_) < TOL, n


def test_workspace_is_checked(device):
    lib = _lib.load()
    B, T, H = 1, 40, 1
    xs = make_inputs(B, T, H, N, seed=9500, dtype=torch.float32)
    need = lib.rwkv7_bwd_workspace_bytes(B, T, H, _lib.DTYPE_F32)
    assert need >= 3 * (2 * 64 * 64 + 2 * 16 * 64) * 4
    rc, _ = run(device, xs, None, None, ws_bytes=need - 256)
    assert rc == -6                     # RWKV7_ERR_WORKSPACE


def test_autograd_of_a_float32_call(device):
    B, T, H = 2, 77, 2
    xs = make_inputs(B, T, H, N, seed=9600, dtype=torch.float32)
    dO, dS = upstream(B, T, H, 6)
    leaves = [x.to(device).requires_grad_(True) for x in xs]
    o, s = rwkv_ops_amd.generalized_delta_rule(*leaves[:6], initial_state=leaves[6])
    ((o * dO.to(device)).sum() + (s * dS.to(device)).sum()).backward()
    ref = orc.gradients(*xs[:6], xs[6], dO, dS)
    for n, leaf, b_ in zip(GRAD_NAMES, leaves, ref):
        assert leaf.grad.dtype == torch.float32
        assert rel_l2(leaf.grad, b_) < TOL, n
