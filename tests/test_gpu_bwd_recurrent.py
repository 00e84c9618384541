"""The float32 recurrent backward (rwkv7_bwd_recurrent) through the C ABI: every dtype it reads, both head sizes,
lengths around the segment (64 / 32 tokens) and block (8 tokens) boundaries, absent upstream gradients and
initial state, against float32 autograd through the CPU oracle on the same rounded inputs.  Tolerances: float32
tensors 1e-4 relative L2 (the forward's float32 tolerance); bf16 / float16 tensors the rounding of the stored
gradient (2^-9 / 2^-11 per element: 4e-3 / 1e-3); dh0 is float32 in every case (1e-4).  And against the chunked
bf16 backward on the same inputs, whose own error is the larger one."""
import pytest
import torch

import rwkv_ops_amd  # noqa: F401  (registers the torch.library ops)

from oracle import rwkv7_native as orc
from rwkv_ops_amd.rwkv7 import _lib
from rwkv_ops_amd.synthetic import GRAD_NAMES, GRAD_TOL, make_inputs, rel_l2

pytestmark = pytest.mark.gpu
CODE = {torch.bfloat16: _lib.DTYPE_BF16, torch.float32: _lib.DTYPE_F32, torch.float16: _lib.DTYPE_F16}
TOL = {torch.float32: 1e-4, torch.bfloat16: 4e-3, torch.float16: 1e-3}


def run(lib, device, xs, dO, dS, N, dtype, entry="rwkv7_bwd_recurrent"):
    B, T, H, _ = xs[0].shape
    dev = [x.to(device) for x in xs[:6]]
    h0 = None if xs[6] is None else xs[6].to(device)
    dO_d = None if dO is None else dO.to(device)
    dS_d = None if dS is None else dS.to(device)
    grads = [torch.full_like(dev[0], float("nan")) for _ in range(6)]
    dh0 = torch.full((B, H, N, N), float("nan"), device=device)
    if entry == "rwkv7_bwd_recurrent":
        size = lib.rwkv7_bwd_recurrent_workspace_bytes(B, T, H, N)
    else:
        size = lib.rwkv7_bwd_workspace_bytes(B, T, H, CODE[dtype])
    ws = torch.empty(size, dtype=torch.uint8, device=device)
    p = lambda t: None if t is None else t.data_ptr()
    rc = getattr(lib, entry)(*[p(x) for x in dev], p(h0), H * N * N, p(dO_d), p(dS_d), *[p(g) for g in grads], p(dh0),
                             B, T, H, N, N, CODE[dtype], p(ws), size, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    return grads + [dh0]


@pytest.mark.parametrize("N,dtype,B,T,H", [
    (64, torch.float32, 2, 1, 2), (64, torch.float32, 1, 7, 1), (64, torch.float32, 2, 63, 2), (64, torch.float32, 1, 64, 3),
    (64, torch.float32, 2, 65, 1), (64, torch.float32, 1, 200, 2), (64, torch.bfloat16, 2, 130, 2), (64, torch.float16, 1, 77, 2),
    (128, torch.float32, 1, 1, 1), (128, torch.float32, 2, 33, 2), (128, torch.float32, 1, 100, 1), (128, torch.bfloat16, 1, 64, 2),
    (128, torch.float16, 2, 40, 1),
    # (every fourth state is kept and a block holds 4 or 8 tokens: lengths around those multiples)
    (128, torch.float32, 1, 2, 1), (128, torch.float32, 1, 3, 2), (128, torch.float32, 2, 35, 1), (128, torch.bfloat16, 1, 6, 1),
    (64, torch.float32, 1, 2, 1), (64, torch.float32, 2, 3, 1), (64, torch.float32, 1, 9, 2), (64, torch.float32, 1, 70, 1)])
def test_recurrent_backward_matches_oracle_autograd(device, N, dtype, B, T, H):
    lib = _lib.load()
    xs = make_inputs(B, T, H, N, seed=3000 + T + N, dtype=dtype)
    g = torch.Generator().manual_seed(T)
    dO = torch.randn(B, T, H, N, generator=g).to(dtype)
    dS = 0.1 * torch.randn(B, H, N, N, generator=g)
    ref = orc.gradients(*xs[:6], xs[6], dO, dS)
    got = run(lib, device, xs, dO, dS, N, dtype)
    errs = {n: rel_l2(a_, b_) for n, a_, b_ in zip(GRAD_NAMES, got, ref)}
    print(f"N={N} {dtype} B={B} T={T} H={H}:", " ".join(f"{k}={v:.2e}" for k, v in errs.items()))
    for n in GRAD_NAMES:
        assert errs[n] < (1e-4 if n == "dh0" else TOL[dtype]), (n, errs)


@pytest.mark.parametrize("N", [64, 128])
def test_recurrent_backward_variants(device, N):
    lib = _lib.load()
    B, T, H = 2, 90, 2
    xs = list(make_inputs(B, T, H, N, seed=3100, dtype=torch.float32))
    g = torch.Generator().manual_seed(3)
    dO = torch.randn(B, T, H, N, generator=g)
    dS = 0.1 * torch.randn(B, H, N, N, generator=g)
    # no gradient into the final state; no gradient into the outputs; no initial state
    for d_o, d_s, h0 in ((dO, None, xs[6]), (None, dS, xs[6]), (dO, dS, None)):
        ys = xs[:6] + [h0]
        ref = orc.gradients(*ys[:6], h0, d_o, d_s)
        got = run(lib, device, ys, d_o, d_s, N, torch.float32)
        for n, a_, b_ in zip(GRAD_NAMES[:6], got, ref):
            assert rel_l2(a_, b_) < 1e-4, (n, d_o is None, d_s is None, h0 is None)
        if h0 is not None:
            assert rel_l2(got[6], ref[6]) < 1e-4
    # padded tail by the w = -1e9 convention: zero gradients there, the rest unchanged
    pad = 20
    mask = torch.ones(B, T, 1, 1)
    mask[:, T - pad:] = 0
    ys = [xs[i] * mask if i != 1 else xs[1] + (1 - mask) * -1e9 for i in range(6)] + [xs[6]]
    got = run(lib, device, ys, dO * mask, dS, N, torch.float32)
    short = run(lib, device, [y[:, :T - pad].contiguous() for y in ys[:6]] + [xs[6]], dO[:, :T - pad].contiguous(), dS, N,
                torch.float32)
    for n, a_, b_ in zip(GRAD_NAMES, got, short):
        if n == "dh0":
            assert rel_l2(a_, b_) < 1e-6
        else:
            assert rel_l2(a_[:, :T - pad], b_) < 1e-6, n
            if n != "dw":
                assert float(a_[:, T - pad:].abs().max()) == 0.0, n


def test_rwkv7_bwd_routes_short_float32_calls_to_the_recurrent_backward(device):
    """A dozen tokens or fewer: rwkv7_bwd on float32 tensors is the recurrent backward, bit for bit; longer calls
    take the chunked float32 backward (tests/test_gpu_bwd_chunk_f32.py), a different order of the same arithmetic."""
    lib = _lib.load()
    N = 64
    for B, T, H, same in ((1, 12, 2, True), (2, 5, 1, True), (1, 100, 2, False)):
        xs = make_inputs(B, T, H, N, seed=3200, dtype=torch.float32)
        g = torch.Generator().manual_seed(4)
        dO = torch.randn(B, T, H, N, generator=g)
        dS = 0.1 * torch.randn(B, H, N, N, generator=g)
        a_ = run(lib, device, xs, dO, dS, N, torch.float32, entry="rwkv7_bwd")
        b_ = run(lib, device, xs, dO, dS, N, torch.float32)
        for x, y in zip(a_, b_):
            assert torch.equal(x, y) if same else rel_l2(x, y) < 1e-5
        if same:
            assert lib.rwkv7_bwd_workspace_bytes(B, T, H, _lib.DTYPE_F32) == lib.rwkv7_bwd_recurrent_workspace_bytes(B, T, H, 64)


def test_recurrent_backward_over_packed_sequences(device):
    """rwkv7_bwd_recurrent_varlen at head size 64 (segments of 64 tokens, their records by (first row / 64) + sequence
    index) against the chunked float32 backward over the same packed float32 rows, and sequence by sequence against
    the dense recurrent call (whose segment states come from the chunked float32 forward, the packed call's from the
    recurrent one: equal to rounding)."""
    lens, H, N = [130, 0, 64, 1, 65, 7], 2, 64
    parts = [make_inputs(1, max(L, 1), H, N, seed=3400 + i, dtype=torch.float32) for i, L in enumerate(lens)]
    parts = [[x[:, :L] for x in p[:6]] + [p[6]] for p, L in zip(parts, lens)]
    packed = [torch.cat([p[j] for p in parts], dim=1).contiguous().to(device) for j in range(6)]
    h0 = torch.cat([p[6] for p in parts], dim=0).contiguous().to(device)
    cu = [0]
    for L in lens:
        cu.append(cu[-1] + L)
    cu_d = torch.tensor(cu, dtype=torch.int32, device=device)
    g = torch.Generator().manual_seed(6)
    dO = torch.randn(1, cu[-1], H, N, generator=g).to(device)
    dS = (0.1 * torch.randn(len(lens), H, N, N, generator=g)).to(device)
    rec = torch.ops.rwkv_ops_amd.rwkv7_bwd_recurrent_varlen(*packed, h0, dO, dS, cu_d)
    chk = torch.ops.rwkv_ops_amd.rwkv7_bwd_varlen(*packed, h0, dO, dS, cu_d)
    for n, x, y in zip(GRAD_NAMES, rec, chk):
        assert rel_l2(x, y) < 1e-5, n
    for i, L in enumerate(lens):
        if L == 0:
            assert torch.equal(rec[6][i], dS[i])
            continue
        one = torch.ops.rwkv_ops_amd.rwkv7_bwd_recurrent(*[x[:, cu[i]:cu[i + 1]].contiguous() for x in packed],
                                                         h0[i:i + 1], dO[:, cu[i]:cu[i + 1]].contiguous(), dS[i:i + 1])
        for j, n in enumerate(GRAD_NAMES):
            mine = rec[j][i:i + 1] if n == "dh0" else rec[j][:, cu[i]:cu[i + 1]]
            assert rel_l2(mine, one[j]) < 2e-6, (i, n)


def test_recurrent_and_chunked_backward_agree(device):
    """bf16 inputs, K = 64: both backward paths on the same inputs; their difference is within the chunked
    kernels' own thresholds."""
    lib = _lib.load()
    B, T, H, N = 2, 300, 3, 64
    xs = make_inputs(B, T, H, N, seed=3300, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(5)
    dO = torch.randn(B, T, H, N, generator=g).to(torch.bfloat16)
    dS = 0.1 * torch.randn(B, H, N, N, generator=g)
    rec = run(lib, device, xs, dO, dS, N, torch.bfloat16)
    chk = run(lib, device, xs, dO, dS, N, torch.bfloat16, entry="rwkv7_bwd")
    for n, x, y in zip(GRAD_NAMES, chk, rec):
        assert rel_l2(x, y) < GRAD_TOL[n], n


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_rwkv7_bwd_takes_head_size_128(device, dtype):
    """rwkv7_bwd and rwkv7_bwd_varlen at K = V = 128 are the token-by-token backward under their own names (with
    its workspace size): the same bits as rwkv7_bwd_recurrent / rwkv7_bwd_recurrent_varlen."""
    lib = _lib.load()
    B, T, H, N = 2, 45, 2, 128
    xs = make_inputs(B, T, H, N, seed=3600, dtype=dtype)
    g = torch.Generator().manual_seed(7)
    dO = torch.randn(B, T, H, N, generator=g).to(dtype)
    dS = 0.1 * torch.randn(B, H, N, N, generator=g)
    ref = run(lib, device, xs, dO, dS, N, dtype)
    dev = [x.to(device) for x in xs[:6]]
    h0, dO_d, dS_d = xs[6].to(device), dO.to(device), dS.to(device)
    p = lambda t: None if t is None else t.data_ptr()
    stream = torch.cuda.current_stream().cuda_stream
    grads = [torch.full_like(dev[0], float("nan")) for _ in range(6)]
    dh0 = torch.full((B, H, N, N), float("nan"), device=device)
    size = lib.rwkv7_bwd_recurrent_workspace_bytes(B, T, H, N)
    ws = torch.empty(size, dtype=torch.uint8, device=device)
    args = (*[p(x) for x in dev], p(h0), H * N * N, p(dO_d), p(dS_d), *[p(x) for x in grads], p(dh0), B, T, H, N, N, CODE[dtype])
    assert lib.rwkv7_bwd(*args, p(ws), size - 256, stream) == -6         # RWKV7_ERR_WORKSPACE
    assert lib.rwkv7_bwd(*args, p(ws), size, stream) == 0
    torch.cuda.synchronize()
    for n, a_, b_ in zip(GRAD_NAMES, grads + [dh0], ref):
        assert torch.equal(a_, b_), n
    # the same rows as one packed row of B sequences
    packed = [x.reshape(1, B * T, H, N) for x in dev]
    cu = torch.tensor([0, T, 2 * T], dtype=torch.int32, device=device)
    want = torch.ops.rwkv_ops_amd.rwkv7_bwd_recurrent_varlen(*packed, h0, dO_d.reshape(1, B * T, H, N), dS_d, cu)
    grads = [torch.full_like(packed[0], float("nan")) for _ in range(6)]
    dh0 = torch.full((B, H, N, N), float("nan"), device=device)
    size = lib.rwkv7_bwd_recurrent_varlen_workspace_bytes(B, B * T, H, N)
    ws = torch.empty(size, dtype=torch.uint8, device=device)
    rc = lib.rwkv7_bwd_varlen(*[p(x) for x in packed], p(cu), B, p(h0), H * N * N, p(dO_d), p(dS_d), *[p(x) for x in grads],
                              p(dh0), B * T, H, N, N, CODE[dtype], p(ws), size, stream)
    assert rc == 0
    torch.cuda.synchronize()
    for n, a_, b_ in zip(GRAD_NAMES, grads + [dh0], want):
        assert torch.equal(a_, b_), n
