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
