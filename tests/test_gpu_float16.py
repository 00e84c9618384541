"""float16 inputs: the decode step and sequences of up to 12 tokens are computed from the float16 values
themselves (RWKV7_DTYPE_F16: decode and recurrent kernels, float32 arithmetic, o rounded to float16); longer
sequences are cast to bfloat16 as the reference's kernel path does (/root/reference/rwkv_ops/rwkv7_kernel/
torch_kernel/torch_op.py:451-455).  Checked against the CPU oracle in float32 on the same rounded inputs:
2e-3 relative L2 on o (float16 rounding of the output: 2^-11 per element), 1e-4 on the state for the native
path; the bf16 tolerance 5e-3 for the cast path."""
import pytest
import torch

import rwkv_ops_amd
from rwkv_ops_amd.rwkv7 import _lib
from oracle import native_c
from rwkv_ops_amd.synthetic import make_inputs, rel_l2

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,T,H,N", [(3, 1, 5, 64), (2, 7, 4, 64), (4, 12, 3, 64), (2, 1, 3, 128), (2, 9, 2, 128)])
def test_float16_native(device, B, T, H, N):
    xs = make_inputs(B, T, H, N, seed=700 + T, dtype=torch.float16)
    o_ref, s_ref = native_c.run(*xs[:6], xs[6])
    dev = [x.to(device) for x in xs]
    o, s = rwkv_ops_amd.generalized_delta_rule(*dev)
    assert o.dtype == torch.float16 and s.dtype == torch.float32
    eo, es = rel_l2(o, o_ref), rel_l2(s, s_ref)
    assert eo < 2e-3 and es < 1e-4, (eo, es)


def test_float16_decode_step_in_place(device):
    B, H = 6, 4
    xs = make_inputs(B, 1, H, 64, seed=711, dtype=torch.float16)
    o_ref, s_ref = native_c.run(*xs[:6], xs[6])
    dev = [x.to(device) for x in xs]
    state = dev[6].clone()
    o = rwkv_ops_amd.rwkv7_decode_step(*[x[:, 0] for x in dev[:6]], state)
    assert o.dtype == torch.float16
    assert rel_l2(o[:, None], o_ref) < 2e-3 and rel_l2(state, s_ref) < 1e-4


def test_float16_long_sequences_take_the_bf16_kernels(device):
    xs = make_inputs(2, 200, 3, 64, seed=712, dtype=torch.float16)
    o_ref, s_ref = native_c.run(*[x.to(torch.bfloat16) for x in xs[:6]], xs[6])
    o, s = rwkv_ops_amd.generalized_delta_rule(*[x.to(device) for x in xs])
    assert o.dtype == torch.float16
    assert rel_l2(o, o_ref) < 5e-3 and rel_l2(s, s_ref) < 5e-3


def test_float16_output_dtype_does_not_depend_on_the_length(device):
    """T = 12 runs the float16 kernels, T = 13 the bf16 chunked ones; `out` is float16 either way, and so is
    the output of a packed call and of a decode step."""
    for T in (1, 12, 13, 100):
        xs = make_inputs(2, T, 3, 64, seed=720 + T, dtype=torch.float16)
        o, s = rwkv_ops_amd.generalized_delta_rule(*[x.to(device) for x in xs])
        assert o.dtype == torch.float16 and s.dtype == torch.float32, T
        ref_in = xs[:6] if T <= 12 else [x.to(torch.bfloat16) for x in xs[:6]]
        o_ref, s_ref = native_c.run(*ref_in, xs[6])
        assert rel_l2(o, o_ref) < 5e-3 and rel_l2(s, s_ref) < 5e-3, T
    xs = make_inputs(1, 90, 3, 64, seed=719, dtype=torch.float16, h0=False)
    o = rwkv_ops_amd.generalized_delta_rule(*[x.to(device) for x in xs[:6]], cu_seqlens=[0, 40, 90],
                                            output_final_state=False)
    assert o.dtype == torch.float16


def test_float16_packed_rows_behind_the_last_sequence(device):
    """rwkv7_fwd_varlen with RWKV7_DTYPE_F16 through the C ABI and a table that ends before T_total: the rows
    of o behind the last sequence are zero-filled -- 2 bytes per element, so the fill ends where o ends (o is
    carved out of a larger buffer of sentinels, which must survive) -- for K = 64 and 128."""
    lib = _lib.load()
    for N in (64, 128):
        T, H, used = 50, 3, 33
        xs = [x.to(device) for x in make_inputs(1, T, H, N, seed=730 + N, dtype=torch.float16, h0=False)[:6]]
        cu = torch.tensor([0, 20, used], dtype=torch.int32, device=device)
        n = T * H * N
        buf = torch.full((3 * n,), 7.0, dtype=torch.float16, device=device)
        o = buf[n:2 * n]
        rc = lib.rwkv7_fwd_varlen(*[x.data_ptr() for x in xs], cu.data_ptr(), 2, None, 0, o.data_ptr(), None,
                                  T, H, N, N, _lib.DTYPE_F16, None, 0, torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        torch.cuda.synchronize()
        assert bool((buf[:n] == 7.0).all()) and bool((buf[2 * n:] == 7.0).all()), "wrote outside o"
        o = o.view(1, T, H, N)
        assert bool((o[:, used:] == 0).all()), "rows behind the last sequence must be zero"
        o_ref, _ = native_c.run(*[x[:, 20:used].cpu() for x in xs], None)
        assert rel_l2(o[:, 20:used], o_ref) < 2e-3


def test_float16_is_refused_where_no_kernel_reads_it(device):
    lib = _lib.load()
    B, T, H = 1, 64, 1
    x = torch.zeros(B, T, H, 64, dtype=torch.float16, device=device)
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device=device)
    p = x.data_ptr()
    assert lib.rwkv7_fwd_chunk_summary(p, p, p, p, p, p, B, T, H, 64, 64, _lib.DTYPE_F16, ws.data_ptr(), ws.numel(), None) == -8
    assert lib.rwkv7_fwd_workspace_bytes(B, T, H, _lib.DTYPE_F16) == 0


def test_float16_gradients_through_the_bf16_backward(device):
    """The backward kernels are bf16: gradients of a float16 call are those of the same call on bf16-cast inputs."""
    xs = make_inputs(2, 8, 3, 64, seed=713, dtype=torch.float16)
    half = [x.to(device).requires_grad_(True) for x in xs[:6]]
    h0 = xs[6].to(device).requires_grad_(True)
    o, s = rwkv_ops_amd.generalized_delta_rule(*half, h0)
    g_o, g_s = torch.randn_like(o, dtype=torch.float32), 0.1 * torch.randn_like(s)
    (o.float() * g_o).sum().add((s * g_s).sum()).backward()
    cast = [x.detach().to(torch.bfloat16).requires_grad_(True) for x in half]
    h0b = h0.detach().clone().requires_grad_(True)
    ob, sb = rwkv_ops_amd.generalized_delta_rule(*cast, h0b)
    (ob.float() * g_o).sum().add((sb * g_s).sum()).backward()
    for a, b in zip(half + [h0], cast + [h0b]):
        assert a.grad is not None and a.grad.dtype == a.dtype and torch.isfinite(a.grad.float()).all()
        assert rel_l2(a.grad.float(), b.grad.float()) < 1e-2
