"""rwkv7_fwd_noalloc: the forward whose workspace is a static device array inside the library, for callers that
cannot allocate.  Called through the C ABI and compared with rwkv7_fwd (caller's workspace) on the same inputs:
bit for bit where both run the one-kernel form (B*H >= 72), within 3e-3 relative L2 where rwkv7_fwd prefers its
two-kernel form (which rounds the per-chunk summaries to bf16 on their way through HBM; measured 1.0e-3), and
against the CPU oracle at the forward's tolerance (5e-3).  Two calls in a row share the array, the second with a smaller input."""
import pytest
import torch

from oracle import native_c
from rwkv_ops_amd.rwkv7 import _lib
from rwkv_ops_amd.synthetic import make_inputs, rel_l2

pytestmark = pytest.mark.gpu


def _both(lib, device, B, T, H, seed, dtype=torch.bfloat16):
    xs = make_inputs(B, T, H, 64, seed=seed, dtype=dtype)
    r, w, k, v, a, b, h0 = [x.to(device) for x in xs]
    code = _lib.DTYPE_BF16 if dtype == torch.bfloat16 else _lib.DTYPE_F32
    stream = torch.cuda.current_stream().cuda_stream
    ptrs = [x.data_ptr() for x in (r, w, k, v, a, b)]
    size = lib.rwkv7_fwd_workspace_bytes(B, T, H, code)
    ws = torch.empty(max(size, 1), dtype=torch.uint8, device=device)
    o1, s1 = torch.empty_like(r), torch.empty(B, H, 64, 64, device=device)
    o2, s2 = torch.full_like(r, float("nan")), torch.full((B, H, 64, 64), float("nan"), device=device)
    rc = lib.rwkv7_fwd(*ptrs, h0.data_ptr(), H * 4096, o1.data_ptr(), s1.data_ptr(), B, T, H, 64, 64, code,
                       ws.data_ptr(), size, stream)
    assert rc == 0
    # everything the second call needs exists by now: between here and the synchronisation nothing is allocated
    before = torch.cuda.memory_stats(device)["allocation.all.allocated"]
    rc = lib.rwkv7_fwd_noalloc(*ptrs, h0.data_ptr(), H * 4096, o2.data_ptr(), s2.data_ptr(), B, T, H, 64, 64, code,
                               stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats(device)["allocation.all.allocated"] == before
    return xs, (o1, s1), (o2, s2)


def test_noalloc_forward_matches_the_workspace_forward(device):
    lib = _lib.load()
    # two calls in a row on the shared array, the second smaller: 128 sequences of 300 tokens, then 96 of 130
    for B, T, H, seed in ((4, 300, 32, 81), (2, 130, 48, 82)):
        xs, (o1, s1), (o2, s2) = _both(lib, device, B, T, H, seed)
        assert torch.equal(o1, o2) and torch.equal(s1, s2), (B, T, H)
        o_ref, s_ref = native_c.run(*xs[:6], xs[6])
        assert rel_l2(o2, o_ref) < 5e-3 and rel_l2(s2, s_ref) < 5e-3
    # below 72 sequences rwkv7_fwd takes two kernels, this entry point still one: smaller again, 6 sequences
    xs, (o1, s1), (o2, s2) = _both(lib, device, 2, 200, 3, 83)
    assert rel_l2(o2, o1) < 3e-3 and rel_l2(s2, s1) < 3e-3
    o_ref, s_ref = native_c.run(*xs[:6], xs[6])
    assert rel_l2(o2, o_ref) < 5e-3 and rel_l2(s2, s_ref) < 5e-3
    # the full 256 sequences the array is sized for, then a decode-sized and a float32 call (no scratch used)
    xs, (o1, s1), (o2, s2) = _both(lib, device, 8, 200, 32, 84)
    assert torch.equal(o1, o2) and torch.equal(s1, s2)
    for B, T, H, dtype in ((3, 1, 5, torch.bfloat16), (2, 7, 4, torch.bfloat16), (2, 40, 3, torch.float32)):
        xs, (o1, s1), (o2, s2) = _both(lib, device, B, T, H, 85, dtype)
        assert torch.equal(o1, o2) and torch.equal(s1, s2), (B, T, H, dtype)


def test_noalloc_forward_refuses_what_does_not_fit(device):
    lib = _lib.load()
    x = torch.zeros(9, 64, 32, 64, dtype=torch.bfloat16, device=device)
    p = x.data_ptr()
    assert lib.rwkv7_fwd_noalloc(p, p, p, p, p, p, None, 0, p, None, 9, 64, 32, 64, 64, 0, None) == -9


@pytest.mark.parametrize("B,H,chunks", [(1, 2, 1100), (2, 3, 530)])
def test_few_heads_and_very_many_chunks_through_the_one_kernel_form(device, B, H, chunks):
    """With a handful of heads the chip holds the workgroups of hundreds of chunk positions of a head at once, so a
    workgroup polls its slot while images many uses old pass through it: the marks of an image (3-bit fields that
    repeat every 7 uses of a slot, the carrier's byte every 255) must tell them apart all the way.  More than 510
    chunks, so that the byte wraps as well.  Against the two-kernel form (which hands no state over through memory)
    and the CPU oracle."""
    lib = _lib.load()
    T = 64 * chunks + 17
    xs, (o1, s1), (o2, s2) = _both(lib, device, B, T, H, 86 + chunks)
    assert torch.isfinite(o2.float()).all() and torch.isfinite(s2).all()
    assert rel_l2(o2, o1) < 3e-3 and rel_l2(s2, s1) < 3e-3
    o_ref, s_ref = native_c.run(*xs[:6], xs[6])
    assert rel_l2(o2, o_ref) < 5e-3 and rel_l2(s2, s_ref) < 5e-3
