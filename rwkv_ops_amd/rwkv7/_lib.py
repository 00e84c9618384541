"""ctypes binding of librwkv7_mi355x.so (the C ABI declared in include/rwkv7_mi355x.h).

The library is built in-tree by ``rwkv_ops_amd/csrc/Makefile``.  There is no other
implementation behind this module: if the shared object is missing, loading raises.
"""
from __future__ import annotations

import ctypes
import os

_CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
LIB_PATH = os.path.join(_CSRC, "librwkv7_mi355x.so")

DTYPE_BF16, DTYPE_F32, DTYPE_F16 = 0, 1, 2
NO_STATUS_RECORD = ctypes.c_size_t(-1).value
FWD_DONE, FWD_GAVE_UP, FWD_NO_LAUNCH = 0, 1, 2
ABI_VERSION = 3

_P, _I, _I64, _SZ = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/rwkv7_mi355x.h and include/rwkv6_mi355x.h one to one
SIGNATURES = {
    "rwkv7_abi_version": (_I, []),
    "rwkv7_status_string": (ctypes.c_char_p, [_I]),
    "rwkv7_fwd_workspace_bytes": (_SZ, [_I, _I, _I, _I]),
    "rwkv7_fwd_status_offset": (_SZ, [_I, _I, _I, _I]),
    "rwkv7_fwd_varlen_status_offset": (_SZ, [_I, _I, _I, _I]),
    "rwkv7_fwd_status": (_I, [_P]),
    "rwkv7_set_giveup_notice": (_I, [_P]),
    "rwkv7_fwd": (_I, [_P] * 6 + [_P, _I64, _P, _P] + [_I] * 6 + [_P, _SZ, _P]),
    "rwkv7_fwd_noalloc": (_I, [_P] * 6 + [_P, _I64, _P, _P] + [_I] * 6 + [_P]),
    "rwkv7_fwd_gather": (_I, [_P] * 6 + [_P, _I, _P, _P, _P] + [_I] * 6 + [_P, _SZ, _P]),
    "rwkv7_decode_step_gather": (_I, [_P] * 6 + [_P, _I, _P, _P, _P] + [_I] * 5 + [_P]),
    "rwkv7_fwd_chunk_workspace_bytes": (_SZ, [_I, _I, _I, _I]),
    "rwkv7_fwd_chunk_summary": (_I, [_P] * 6 + [_I] * 6 + [_P, _SZ, _P]),
    "rwkv7_fwd_chunk_scan": (_I, [_P, _I64, _P, _P] + [_I] * 6 + [_P, _SZ, _P]),
    "rwkv7_bwd_workspace_bytes": (_SZ, [_I, _I, _I, _I]),
    "rwkv7_bwd": (_I, [_P] * 6 + [_P, _I64, _P, _P] + [_P] * 7 + [_I] * 6 + [_P, _SZ, _P]),
    "rwkv7_bwd_recurrent_workspace_bytes": (_SZ, [_I, _I, _I, _I]),
    "rwkv7_bwd_recurrent": (_I, [_P] * 6 + [_P, _I64, _P, _P] + [_P] * 7 + [_I] * 6 + [_P, _SZ, _P]),
    "rwkv7_fwd_varlen_workspace_bytes": (_SZ, [_I, _I, _I, _I]),
    "rwkv7_fwd_varlen": (_I, [_P] * 6 + [_P, _I, _P, _I64, _P, _P] + [_I] * 5 + [_P, _SZ, _P]),
    "rwkv7_bwd_varlen_workspace_bytes": (_SZ, [_I, _I, _I, _I]),
    "rwkv7_bwd_varlen": (_I, [_P] * 6 + [_P, _I, _P, _I64, _P, _P] + [_P] * 7 + [_I] * 5 + [_P, _SZ, _P]),
    "rwkv7_bwd_recurrent_varlen_workspace_bytes": (_SZ, [_I, _I, _I, _I]),
    "rwkv7_bwd_recurrent_varlen": (_I, [_P] * 6 + [_P, _I, _P, _I64, _P, _P] + [_P] * 7 + [_I] * 5 + [_P, _SZ, _P]),
    "rwkv6_fwd_workspace_bytes": (_SZ, [_I, _I, _I, _I]),
    "rwkv6_fwd": (_I, [_P] * 5 + [_P, _I, _P, _P, _P] + [_I] * 6 + [_P, _SZ, _P]),
    "rwkv6_bwd_workspace_bytes": (_SZ, [_I, _I, _I, _I]),
    "rwkv6_bwd_workspace_bytes_head": (_SZ, [_I, _I, _I, _I, _I]),
    "rwkv6_bwd": (_I, [_P] * 6 + [_P] * 5 + [_I] * 6 + [_P, _SZ, _P]),
    "rwkv6_fwd_recurrent": (_I, [_P] * 5 + [_P, _I, _P, _P, _P] + [_I] * 6 + [_P]),
    "rwkv7_fwd_recurrent": (_I, [_P] * 6 + [_P, _I64, _P, _P] + [_I] * 6 + [_P]),
    "rwkv7_decode_step": (_I, [_P] * 6 + [_P, _I64, _P, _P] + [_I] * 5 + [_P]),
}

_lib = None


class Rwkv7LibraryError(RuntimeError):
    pass


def load():
    """Loads the shared library once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise Rwkv7LibraryError(
            f"{LIB_PATH} is missing: build it with `make -C {_CSRC}` "
            "(there is no fallback implementation)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    if lib.rwkv7_abi_version() != ABI_VERSION:
        raise Rwkv7LibraryError(
            f"{LIB_PATH} has ABI version {lib.rwkv7_abi_version()}, expected {ABI_VERSION}; rebuild it")
    _lib = lib
    return lib


_notice = None          # one pinned int64 word that a fused forward which gives up writes into


def giveup_notice():
    """The pinned host word registered with ``rwkv7_set_giveup_notice`` (allocated and registered on first use)."""
    global _notice
    if _notice is None:
        import torch
        word = torch.zeros(1, dtype=torch.int64).pin_memory()
        check(load().rwkv7_set_giveup_notice(word.data_ptr()), "rwkv7_set_giveup_notice")
        _notice = word
    return _notice


class ForwardGaveUp(RuntimeError):
    """A one-kernel chunked forward stopped waiting for the state of the chunk before (its outputs hold NaN)."""


def raise_if_gave_up() -> None:
    """Looks at the notice word: a plain read of pinned host memory, no synchronisation.  A forward that gave
    up earlier (in any stream) is reported by the first call that comes after the device's store has landed."""
    if _notice is None:
        import torch
        # (the word is pinned memory: not to be allocated while a graph is being captured; the first call
        # outside a capture registers it)
        if torch.cuda.is_available() and torch.cuda.is_current_stream_capturing():
            return
    word = giveup_notice()
    if int(word[0]) != 0:
        word[0] = 0
        raise ForwardGaveUp(
            "an earlier rwkv7 forward gave up: a workgroup waited two seconds for the state of the chunk before it "
            "and filled its outputs with NaN (see rwkv7_fwd_status in include/rwkv7_mi355x.h)")


def status_string(status: int) -> str:
    return load().rwkv7_status_string(int(status)).decode()


def check(status: int, what: str) -> None:
    """0 -> ok; argument errors (< 0) -> ValueError; launch errors (> 0) -> RuntimeError."""
    if status == 0:
        return
    msg = f"{what}: {status_string(status)} (status {status})"
    if status < 0:
        raise ValueError(msg)
    raise RuntimeError(msg)
