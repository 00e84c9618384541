"""CPU checks of the C ABI: the library loads without a GPU, exports every symbol the
header declares, and rejects bad arguments with the documented status before any launch."""
import ctypes
import os
import re

import pytest

from rwkv_ops_amd.rwkv7 import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", "rwkv7_mi355x.h"), os.path.join(ROOT, "include", "rwkv6_mi355x.h")]


def declared_functions():
    text = "".join(open(h).read() for h in HEADERS)
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rwkv[67]_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    names = declared_functions()
    assert names, "no declarations parsed"
    assert sorted(_lib.SIGNATURES) == names


def test_every_declared_symbol_is_exported():
    lib = _lib.load()
    for name in declared_functions():
        assert hasattr(lib, name), name
    assert lib.rwkv7_abi_version() == _lib.ABI_VERSION


def test_status_strings():
    for code in range(-9, 1):
        s = _lib.status_string(code)
        assert s and "unknown" not in s
    assert "unknown" in _lib.status_string(-99)


P = ctypes.c_void_p


def _call_fwd(lib, ptrs=None, h0=None, stride=0, o=0x1000, ht=None, B=1, T=4, H=2, K=64, V=64, dtype=0,
              ws=None, ws_bytes=0):
    ptrs = ptrs or [0x1000] * 6
    return lib.rwkv7_fwd(*ptrs, h0, stride, o, ht, B, T, H, K, V, dtype, ws, ws_bytes, None)


def test_argument_errors_do_not_launch():
    lib = _lib.load()
    assert _call_fwd(lib, dtype=7) == -2
    assert _call_fwd(lib, K=128) == -3
    assert _call_fwd(lib, V=32) == -3
    assert _call_fwd(lib, B=0) == -4
    assert _call_fwd(lib, T=0) == -4
    assert _call_fwd(lib, ptrs=[0x1000, None, 0x1000, 0x1000, 0x1000, 0x1000]) == -1
    assert _call_fwd(lib, o=None) == -1
    assert _call_fwd(lib, h0=0x2000, stride=17) == -5
    assert _call_fwd(lib, ptrs=[0x1004] + [0x1000] * 5) == -7
    rc = lib.rwkv7_decode_step(*[0x1000] * 6, None, 0, 0x1000, None, 1, 1, 64, 32, 0, None)
    assert rc == -3
    # K = V = 128: the backward hands it to the token-by-token kernel (which asks for its workspace); the
    # two-kernel entry points refuse it
    rc = lib.rwkv7_bwd(*[0x1000] * 6, None, 0, None, None, *[0x1000] * 6, None, 1, 4, 2, 128, 128, 0, None, 0, None)
    assert rc == -6
    assert lib.rwkv7_bwd_recurrent_workspace_bytes(1, 4, 2, 128) > 0
    rc = lib.rwkv7_fwd_chunk_summary(*[0x1000] * 6, 1, 4, 2, 128, 128, 0, None, 0, None)
    assert rc == -3
    assert _call_fwd(lib, K=256, V=256) == -3
    rc = lib.rwkv7_fwd_recurrent(*[0x1000] * 6, None, 0, None, None, 1, 1, 1, 64, 64, 1, None)
    assert rc == -1


def test_check_maps_status_to_exceptions():
    with pytest.raises(ValueError):
        _lib.check(-3, "x")
    with pytest.raises(RuntimeError):
        _lib.check(1, "x")
    _lib.check(0, "x")


def test_varlen_argument_errors_do_not_launch():
    lib = _lib.load()

    def fwd(cu=0x3000, n_seq=2, T=100, H=2, K=64, dtype=0, ws=None, ws_bytes=0, r=0x1000):
        return lib.rwkv7_fwd_varlen(r, *[0x1000] * 5, cu, n_seq, None, 0, 0x1000, None, T, H, K, 64, dtype,
                                    ws, ws_bytes, None)
    assert fwd(cu=None) == -1
    assert fwd(cu=0x3002) == -7
    assert fwd(n_seq=0) == -4
    assert fwd(T=0) == -4
    assert fwd(K=128) == -3
    assert fwd(dtype=5) == -2
    assert fwd(r=None) == -1
    assert fwd() == -6                                   # bf16 needs a workspace
    # the workspace covers T / 64 + n_seq chunks per head, whatever the lengths turn out to be
    n_seq, T, H = 5, 1000, 3
    chunks = (T // 64 + n_seq) * H
    assert lib.rwkv7_fwd_varlen_workspace_bytes(n_seq, T, H, 0) >= chunks * (4 * 8192 + 256)
    assert lib.rwkv7_bwd_varlen_workspace_bytes(n_seq, T, H, 0) >= chunks * (3 * 8192 + 256 + 2 * 16384)
    assert lib.rwkv7_fwd_varlen_workspace_bytes(n_seq, T, H, 1) == 0
    assert lib.rwkv7_fwd_varlen_workspace_bytes(64, T, H, 0) < 64 * H * 40000   # one-kernel form: no per-chunk records
    rc = lib.rwkv7_bwd_varlen(*[0x1000] * 6, 0x3000, 2, None, 0, None, None, *[0x1000] * 6, None,
                              100, 2, 64, 64, 1, None, 0, None)
    assert rc == -6                                      # float32 rows: the chunked float32 backward, which needs
    # 40 KiB per 16 tokens (T / 16 + n_seq records per head) and 1 MiB per sequence-head, up to 1024 of them
    assert lib.rwkv7_bwd_varlen_workspace_bytes(n_seq, T, H, 1) >= (T // 16 + n_seq) * H * 40960 + n_seq * H * (1 << 20)
    assert lib.rwkv7_bwd_varlen_workspace_bytes(2000, 20000, 4, 1) < (20000 // 16 + 2000) * 4 * 40960 + 1025 * (1 << 20)
    rc = lib.rwkv7_bwd_varlen(*[0x1000] * 6, 0x3000, 2, None, 0, None, None, *[0x1000] * 6, None,
                              100, 2, 128, 128, 1, None, 0, None)
    assert rc == -6                                      # head size 128: the token-by-token backward's workspace
    rc = lib.rwkv7_bwd_varlen(*[0x1000] * 6, None, 2, None, 0, None, None, *[0x1000] * 6, None,
                              100, 2, 64, 64, 0, None, 0, None)
    assert rc == -1


def test_rwkv6_argument_errors_do_not_launch():
    lib = _lib.load()
    x = 0x1000

    def fwd(u=x, states=None, n_state=0, smap=None, B=2, T=100, K=64, dtype=0, r=x):
        return lib.rwkv6_fwd(r, x, x, x, u, states, n_state, smap, x, None, B, T, 2, K, 64, dtype, None, 0, None)
    assert fwd(u=None) == -1
    assert fwd(r=None) == -1
    assert fwd(K=32) == -3
    assert fwd(dtype=3) == -2
    assert fwd(smap=0x2000) == -1                        # a map without states
    assert fwd(states=0x4000, n_state=3) == -4           # neither shared (1) nor one per row (B): needs a map
    assert fwd(states=0x4000, n_state=0, smap=0x2000) == -4
    assert fwd() == -6                                   # bf16, T > 1: workspace required
    assert lib.rwkv6_fwd_workspace_bytes(2, 100, 2, 0) == lib.rwkv7_fwd_workspace_bytes(2, 100, 2, 0)

    def bwd(u=x, dy=x, du=x, dtype=0, ws=None, ws_bytes=0):
        return lib.rwkv6_bwd(x, x, x, x, u, dy, x, x, x, x, du, 2, 100, 2, 64, 64, dtype, ws, ws_bytes, None)
    assert bwd(dtype=2) == -8                            # float16 backward is not built
    assert bwd(dtype=1) == -6                            # float32: built, and it wants its workspace
    assert bwd(u=None) == -1 and bwd(dy=None) == -1 and bwd(du=None) == -1
    assert bwd() == -6
    assert lib.rwkv6_bwd_workspace_bytes(2, 8, 2, 0) > 3 * 2 * 8 * 2 * 64 * 2
    assert lib.rwkv6_bwd_workspace_bytes(2, 8, 2, 1) > 3 * 2 * 8 * 2 * 64 * 4
    assert lib.rwkv6_bwd_workspace_bytes(2, 8, 2, 2) == 0
    # the head size as an argument: 64 is the plain function, 128 is built (larger tensors), others are not
    assert lib.rwkv6_bwd_workspace_bytes_head(2, 8, 2, 64, 0) == lib.rwkv6_bwd_workspace_bytes(2, 8, 2, 0)
    assert lib.rwkv6_bwd_workspace_bytes_head(2, 8, 2, 128, 0) > 3 * 2 * 8 * 2 * 128 * 2
    assert lib.rwkv6_bwd_workspace_bytes_head(2, 8, 2, 128, 1) > 3 * 2 * 8 * 2 * 128 * 4
    assert lib.rwkv6_bwd_workspace_bytes_head(2, 8, 2, 96, 0) == 0
    assert fwd(K=128) == -3                              # K = 128 against V = 64


def test_float16_is_a_dtype_only_where_a_kernel_reads_it():
    """RWKV7_DTYPE_F16 (2): accepted by the entry points that reach the decode step or the recurrent forward
    (their argument checks pass and fail as for the other dtypes), 'not built' (-8) everywhere else, and no
    workspace size exists for it.  No launch happens: every call below stops at an argument check."""
    lib = _lib.load()
    x = 0x1000
    assert _lib.DTYPE_F16 == 2
    assert lib.rwkv7_fwd_chunk_summary(x, x, x, x, x, x, 1, 64, 1, 64, 64, 2, x, 1 << 20, None) == -8
    assert lib.rwkv7_bwd(x, x, x, x, x, x, None, 0, x, None, x, x, x, x, x, x, x, 1, 64, 1, 64, 64, 2, x, 1 << 20, None) == -8
    assert lib.rwkv6_fwd(x, x, x, x, x, None, 0, None, x, None, 2, 100, 2, 64, 64, 2, None, 0, None) == -8
    for fn in (lib.rwkv7_fwd_workspace_bytes, lib.rwkv7_fwd_chunk_workspace_bytes, lib.rwkv7_bwd_workspace_bytes):
        assert fn(2, 100, 2, 2) == 0
    # accepted as a dtype by the decode step: the next check (head size, null pointer) is what answers
    assert lib.rwkv7_decode_step(x, x, x, x, x, x, None, 0, x, None, 2, 2, 32, 32, 2, None) == -3
    assert lib.rwkv7_decode_step(None, x, x, x, x, x, None, 0, x, None, 2, 2, 64, 64, 2, None) == -1


def test_forward_status_record_on_a_host_image():
    """rwkv7_fwd_status reads a HOST copy of the 16-byte record [flag, tag] that a chunked forward leaves in
    its workspace; the offsets of the record lie inside the workspace of the form the call would choose."""
    lib = _lib.load()
    rec = (ctypes.c_uint64 * 2)

    def status(flag, tag):
        return lib.rwkv7_fwd_status(ctypes.cast(rec(flag, tag), ctypes.c_void_p))
    assert status(0, 0) == _lib.FWD_NO_LAUNCH                        # a fresh (zeroed) workspace
    tag = 0x9e3779b97f4a7c15
    assert status(tag - 1, tag) == _lib.FWD_DONE                     # what the first workgroup writes
    assert status(tag, tag) == _lib.FWD_GAVE_UP                      # what a wave that stopped waiting writes
    assert status(12345, tag) == _lib.FWD_DONE                       # anything but the tag itself
    assert lib.rwkv7_fwd_status(None) == -1
    # a workspace image built on the host: zeros, then the record of a finished launch at the documented offset
    for B, T, H in ((8, 4096, 32), (1, 300, 4)):                     # one-kernel form, two-kernel form
        size = lib.rwkv7_fwd_workspace_bytes(B, T, H, 0)
        off = lib.rwkv7_fwd_status_offset(B, T, H, 0)
        assert off % 16 == 0 and off + 16 <= size
        image = bytearray(size)
        view = (ctypes.c_char * size).from_buffer(image)
        assert lib.rwkv7_fwd_status(ctypes.cast(ctypes.addressof(view) + off, ctypes.c_void_p)) == _lib.FWD_NO_LAUNCH
        image[off:off + 16] = (tag - 1).to_bytes(8, "little") + tag.to_bytes(8, "little")
        assert lib.rwkv7_fwd_status(ctypes.cast(ctypes.addressof(view) + off, ctypes.c_void_p)) == _lib.FWD_DONE
        image[off:off + 8] = tag.to_bytes(8, "little")
        assert lib.rwkv7_fwd_status(ctypes.cast(ctypes.addressof(view) + off, ctypes.c_void_p)) == _lib.FWD_GAVE_UP
        del view
    n_seq, T, H = 5, 1000, 32
    off = lib.rwkv7_fwd_varlen_status_offset(n_seq, T, H, 0)
    assert off % 16 == 0 and off + 16 <= lib.rwkv7_fwd_varlen_workspace_bytes(n_seq, T, H, 0)
    # calls that run no chunked kernel leave no record
    assert lib.rwkv7_fwd_status_offset(8, 12, 32, 0) == _lib.NO_STATUS_RECORD
    assert lib.rwkv7_fwd_status_offset(8, 4096, 32, 1) == _lib.NO_STATUS_RECORD
    assert lib.rwkv7_fwd_varlen_status_offset(5, 1000, 32, 2) == _lib.NO_STATUS_RECORD


def test_noalloc_forward_argument_errors_do_not_launch():
    lib = _lib.load()
    x = 0x1000

    def fwd(B=8, T=100, H=32, K=64, dtype=0, r=x, o=x):
        return lib.rwkv7_fwd_noalloc(r, x, x, x, x, x, None, 0, o, None, B, T, H, K, K, dtype, None)
    assert fwd(B=9) == -9                                            # 288 sequences: beyond the static scratch
    assert fwd(B=1, H=257) == -9
    assert "256" in _lib.status_string(-9)
    assert fwd(r=None) == -1 and fwd(o=None) == -1
    assert fwd(K=32) == -3
    assert fwd(dtype=9) == -2
    assert fwd(T=0) == -4
