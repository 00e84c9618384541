"""The status record of a chunked forward (rwkv7_fwd_status): after a normal call, in either form, through the
C ABI, the record read back from the workspace says that the launch ran and did not give up."""
import ctypes

import pytest
import torch

from rwkv_ops_amd.rwkv7 import _lib
from rwkv_ops_amd.synthetic import make_inputs

pytestmark = pytest.mark.gpu


def _status(lib, ws, off):
    rec = ws[off:off + 16].cpu().numpy().tobytes()
    buf = ctypes.create_string_buffer(rec, 16)
    return lib.rwkv7_fwd_status(ctypes.cast(buf, ctypes.c_void_p)), rec


@pytest.mark.parametrize("B,T,H", [(4, 300, 32), (1, 300, 4)])          # one-kernel form, two-kernel form
def test_status_after_a_normal_forward(device, B, T, H):
    lib = _lib.load()
    r, w, k, v, a, b, h0 = [x.to(device) for x in make_inputs(B, T, H, 64, seed=71, dtype=torch.bfloat16)]
    size = lib.rwkv7_fwd_workspace_bytes(B, T, H, 0)
    off = lib.rwkv7_fwd_status_offset(B, T, H, 0)
    ws = torch.zeros(size, dtype=torch.uint8, device=device)
    assert _status(lib, ws, off)[0] == _lib.FWD_NO_LAUNCH
    o = torch.empty_like(r)
    ht = torch.empty(B, H, 64, 64, device=device)
    tags = []
    for _ in range(2):
        rc = lib.rwkv7_fwd(*[x.data_ptr() for x in (r, w, k, v, a, b)], h0.data_ptr(), H * 4096, o.data_ptr(),
                           ht.data_ptr(), B, T, H, 64, 64, 0, ws.data_ptr(), size,
                           torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        torch.cuda.synchronize()
        st, rec = _status(lib, ws, off)
        assert st == _lib.FWD_DONE
        tags.append(rec[8:])
        assert torch.isfinite(o.float()).all() and torch.isfinite(ht).all()
    assert tags[0] != tags[1]                                            # every launch draws a new tag


def test_status_after_a_packed_forward(device):
    lib = _lib.load()
    T, H = 700, 32
    r, w, k, v, a, b, _ = [None if x is None else x.to(device)
                           for x in make_inputs(1, T, H, 64, seed=72, dtype=torch.bfloat16, h0=False)]
    cu = torch.tensor([0, 100, 100, 350, 700], dtype=torch.int32, device=device)
    n_seq = 4
    size = lib.rwkv7_fwd_varlen_workspace_bytes(n_seq, T, H, 0)
    off = lib.rwkv7_fwd_varlen_status_offset(n_seq, T, H, 0)
    ws = torch.zeros(size, dtype=torch.uint8, device=device)
    o = torch.empty_like(r)
    rc = lib.rwkv7_fwd_varlen(*[x.data_ptr() for x in (r, w, k, v, a, b)], cu.data_ptr(), n_seq, None, 0,
                              o.data_ptr(), None, T, H, 64, 64, 0, ws.data_ptr(), size,
                              torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert _status(lib, ws, off)[0] == _lib.FWD_DONE


def test_giveup_notice_reaches_python(device):
    """The pinned host word that a forward which gives up writes into: the next forward call raises, the call
    after it runs (the word is cleared by the look), and ``last_forward_status`` reports and clears it too.
    No wait is made to time out on the GPU: the host plays the device's part and sets the word."""
    import rwkv_ops_amd
    xs = [x.to(device) for x in make_inputs(2, 200, 48, 64, seed=73, dtype=torch.bfloat16)]
    o, s = rwkv_ops_amd.generalized_delta_rule(*xs)                       # registers the word on first use
    assert rwkv_ops_amd.last_forward_status(synchronize=True) == "ok"
    word = _lib.giveup_notice()
    assert word.is_pinned() and int(word[0]) == 0
    word[0] = 12345
    with pytest.raises(_lib.ForwardGaveUp):
        rwkv_ops_amd.generalized_delta_rule(*xs)
    o2, s2 = rwkv_ops_amd.generalized_delta_rule(*xs)
    assert torch.equal(o2, o) and torch.equal(s2, s)
    word[0] = 7
    assert rwkv_ops_amd.last_forward_status() == "gave_up"
    assert rwkv_ops_amd.last_forward_status() == "ok"


def test_the_device_can_write_the_notice_word(device):
    """The word is host memory that kernels can store to: a device-side fill of a view of it is seen by the host."""
    word = _lib.giveup_notice()
    word[0] = 0
    import ctypes as c
    hip = c.CDLL("libamdhip64.so")
    dev_ptr = c.c_void_p()
    assert hip.hipHostGetDevicePointer(c.byref(dev_ptr), c.c_void_p(word.data_ptr()), 0) == 0
    assert dev_ptr.value == word.data_ptr()          # the same address on both sides: what the library is given
    assert hip.hipMemsetD32(dev_ptr, 0x01010101, 2) == 0
    torch.cuda.synchronize()
    assert int(word[0]) == 0x0101010101010101
    word[0] = 0
