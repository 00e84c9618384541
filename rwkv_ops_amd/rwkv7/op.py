"""`generalized_delta_rule` for MI355X: the host side of the drop-in.

Mirrors the operator interface of the reference's kernel path
(/root/reference/rwkv_ops/rwkv7_kernel/torch_op.py:458-490): same positional order
``(r, w, k, v, a, b)``, same keywords and defaults, same ``[B, T, H, K]`` /
``head_first`` layouts, ``initial_state [N, H, K, V]``, and the same return
convention (``(out, state)`` when ``output_final_state`` else the bare ``out``,
torch_op.py:487-490).  The work is done by ``torch.library`` custom ops that call the
C ABI of librwkv7_mi355x.so on the current HIP stream.

Deliberate differences from the reference's Triton path, both towards its own native
path (/root/reference/rwkv_ops/rwkv7_kernel/native_keras_op.py):
  * float32 inputs are computed in float32 and return a float32 ``out`` (the Triton
    path casts everything to bfloat16, torch_op.py:451-455);
  * the final state is returned in float32 (native_keras_op.py:94), not cast to the
    input dtype (torch_op.py:488), so that a decode loop can feed it back losslessly;
  * an ``initial_state`` with N == 1 is broadcast over the batch
    (native_keras_op.py:62-63).
One addition: ``state_map`` (int tensor or list ``[B]``) lets batch row b start from
``initial_state[state_map[b]]``, ``initial_state`` then being ``[n_state, H, K, V]`` -- the
facility the reference's RWKV6 operator has
(/root/reference/rwkv_ops/rwkv6_kernel/torch_rwkv_kernel.py:259-298) and its RWKV7 one lacks.
And ``cu_seqlens``, which the reference declares on ``chunk_dplr_delta_rule`` with its checks
(torch_op.py:338,363-365,388-398) but neither exposes on ``generalized_delta_rule`` nor hands to its
kernels: sequences of different lengths packed into one batch row, one state per sequence.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib

HEAD_SIZE = 64
# K = V = 128 has the decode step, a chunked bf16 forward of its own and the float32 recurrent forward and backward
HEAD_SIZES = (64, 128)

__all__ = ["generalized_delta_rule", "rwkv7_decode_step", "last_forward_status", "HEAD_SIZE"]


def _dtype_code(dt: torch.dtype) -> int:
    if dt == torch.bfloat16:
        return _lib.DTYPE_BF16
    if dt == torch.float32:
        return _lib.DTYPE_F32
    if dt == torch.float16:
        return _lib.DTYPE_F16
    raise ValueError(f"unsupported compute dtype {dt}")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _require_gpu(t: torch.Tensor) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            "rwkv_ops_amd runs on MI355X only: tensors must live on a ROCm device "
            f"(got {t.device}); there is no CPU implementation behind this operator")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_ptr(device: torch.device) -> int:
    """The current stream of ``device`` as a ``hipStream_t`` value."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)            # the same handle, without building a Stream object
    return torch.cuda.current_stream(device).cuda_stream


class _on_device:
    """``torch.cuda.device(dev)`` only when ``dev`` is not already the current device."""
    __slots__ = ("ctx",)

    def __init__(self, dev: torch.device):
        self.ctx = None if dev.index == torch.cuda.current_device() else torch.cuda.device(dev)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            return self.ctx.__exit__(*exc)
        return False


def _h0_stride(h0: Optional[torch.Tensor], B: int, H: int) -> int:
    if h0 is None:
        return 0
    return 0 if (h0.shape[0] == 1 and B != 1) else H * h0.shape[-1] * h0.shape[-2]


# --------------------------------------------------------------------------- custom ops
def _direct(*tensors) -> bool:
    """True when a call may go straight to the library: not under torch.compile, and nothing to
    differentiate.  The torch.library dispatcher costs about 10 us per call, which is more than a small
    decode step takes on the GPU."""
    if torch.compiler.is_compiling():
        return False
    if torch.is_grad_enabled():
        for t in tensors:
            if t is not None and t.requires_grad:
                return False
    return True


def last_forward_status(synchronize: bool = False) -> str:
    """"ok" or "gave_up": whether a one-kernel chunked forward launched from this process has stopped waiting for
    a state hand-off and poisoned its outputs with NaN since the last look (the look clears the mark).  Reads one
    word of pinned host memory; with ``synchronize`` the devices are synchronised first, so that every forward
    launched so far has had its say.  The forward calls look themselves, at their start, and raise
    ``ForwardGaveUp`` -- this function is for a caller that wants to know before its next call."""
    if synchronize and torch.cuda.is_available():
        torch.cuda.synchronize()
    word = _lib.giveup_notice()
    gave_up = int(word[0]) != 0
    word[0] = 0
    return "gave_up" if gave_up else "ok"


def _fwd_impl(r, w, k, v, a, b, h0, want_state, state_map=None):
    lib = _lib.load()
    _lib.raise_if_gave_up()
    B, T, H, N = r.shape
    o = torch.empty_like(r)
    ht = torch.empty((B, H, N, N) if want_state else (0,), dtype=torch.float32, device=r.device)
    code = _dtype_code(r.dtype)
    with _on_device(r.device):
        ws_bytes = lib.rwkv7_fwd_workspace_bytes(B, T, H, code)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=r.device) if ws_bytes else None
        if state_map is None:
            rc = lib.rwkv7_fwd(_ptr(r), _ptr(w), _ptr(k), _ptr(v), _ptr(a), _ptr(b),
                               _ptr(h0), _h0_stride(h0, B, H), _ptr(o), _ptr(ht) if want_state else None,
                               B, T, H, N, N, code, _ptr(ws), ws_bytes, _stream_ptr(r.device))
        else:
            rc = lib.rwkv7_fwd_gather(_ptr(r), _ptr(w), _ptr(k), _ptr(v), _ptr(a), _ptr(b),
                                      _ptr(h0), h0.shape[0], _ptr(state_map), _ptr(o),
                                      _ptr(ht) if want_state else None,
                                      B, T, H, N, N, code, _ptr(ws), ws_bytes, _stream_ptr(r.device))
    _lib.check(rc, "rwkv7_fwd")
    return o, ht


@torch.library.custom_op("rwkv_ops_amd::rwkv7_fwd", mutates_args=(), device_types="cuda")
def rwkv7_fwd(r: torch.Tensor, w: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
              a: torch.Tensor, b: torch.Tensor, h0: Optional[torch.Tensor],
              want_state: bool, state_map: Optional[torch.Tensor] = None
              ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Inputs ``[B, T, H, 64]`` contiguous, one dtype (bf16 or f32); ``h0`` float32
    ``[B or 1, H, 64, 64]`` contiguous or None -- or ``[n_state, H, 64, 64]`` with
    ``state_map`` int32 ``[B]``.  Returns ``(o, ht)``; ``ht`` is an empty tensor when
    ``want_state`` is false."""
    return _fwd_impl(r, w, k, v, a, b, h0, want_state, state_map)


@rwkv7_fwd.register_fake
def _(r, w, k, v, a, b, h0, want_state, state_map=None):
    B, T, H, N = r.shape
    return torch.empty_like(r), r.new_empty((B, H, N, N) if want_state else (0,), dtype=torch.float32)


@torch.library.custom_op("rwkv_ops_amd::rwkv7_bwd", mutates_args=(), device_types="cuda")
def rwkv7_bwd(r: torch.Tensor, w: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
              a: torch.Tensor, b: torch.Tensor, h0: Optional[torch.Tensor],
              d_o: Optional[torch.Tensor], d_ht: Optional[torch.Tensor]
              ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor,
                         torch.Tensor, torch.Tensor]:
    """Gradients of ``rwkv7_fwd``: bf16 or float32 ``[B, T, H, 64]`` inputs (contiguous), ``d_o`` like ``r`` or
    None, ``d_ht`` float32 ``[B, H, 64, 64]`` or None.  Returns ``(dr, dw, dk, dv, da, db, dh0)`` with
    ``dh0`` float32 ``[B, H, 64, 64]`` (per batch entry, also when ``h0`` is a broadcast ``[1, ...]``)."""
    lib = _lib.load()
    B, T, H, N = r.shape
    code = _dtype_code(r.dtype)
    grads = [torch.empty_like(r) for _ in range(6)]
    dh0 = torch.empty((B, H, N, N), dtype=torch.float32, device=r.device)
    with _on_device(r.device):
        ws_bytes = lib.rwkv7_bwd_workspace_bytes(B, T, H, code)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=r.device)
        rc = lib.rwkv7_bwd(_ptr(r), _ptr(w), _ptr(k), _ptr(v), _ptr(a), _ptr(b),
                           _ptr(h0), _h0_stride(h0, B, H), _ptr(d_o), _ptr(d_ht),
                           *[_ptr(x) for x in grads], _ptr(dh0),
                           B, T, H, N, N, code, _ptr(ws), ws_bytes, _stream_ptr(r.device))
    _lib.check(rc, "rwkv7_bwd")
    return (*grads, dh0)


@rwkv7_bwd.register_fake
def _(r, w, k, v, a, b, h0, d_o, d_ht):
    B, T, H, N = r.shape
    return tuple(torch.empty_like(r) for _ in range(6)) + (r.new_empty((B, H, N, N), dtype=torch.float32),)


@torch.library.custom_op("rwkv_ops_amd::rwkv7_bwd_recurrent", mutates_args=(), device_types="cuda")
def rwkv7_bwd_recurrent(r: torch.Tensor, w: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                        a: torch.Tensor, b: torch.Tensor, h0: Optional[torch.Tensor],
                        d_o: Optional[torch.Tensor], d_ht: Optional[torch.Tensor]
                        ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor,
                                   torch.Tensor, torch.Tensor]:
    """Gradients of ``rwkv7_fwd`` from the float32 recurrent backward: any of the three dtypes, head size 64
    or 128; same arguments and results as ``rwkv7_bwd`` (gradients in the dtype of the inputs)."""
    lib = _lib.load()
    B, T, H, N = r.shape
    grads = [torch.empty_like(r) for _ in range(6)]
    dh0 = torch.empty((B, H, N, N), dtype=torch.float32, device=r.device)
    with _on_device(r.device):
        ws_bytes = lib.rwkv7_bwd_recurrent_workspace_bytes(B, T, H, N)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=r.device)
        rc = lib.rwkv7_bwd_recurrent(_ptr(r), _ptr(w), _ptr(k), _ptr(v), _ptr(a), _ptr(b),
                                     _ptr(h0), _h0_stride(h0, B, H), _ptr(d_o), _ptr(d_ht),
                                     *[_ptr(x) for x in grads], _ptr(dh0),
                                     B, T, H, N, N, _dtype_code(r.dtype), _ptr(ws), ws_bytes, _stream_ptr(r.device))
    _lib.check(rc, "rwkv7_bwd_recurrent")
    return (*grads, dh0)


@rwkv7_bwd_recurrent.register_fake
def _(r, w, k, v, a, b, h0, d_o, d_ht):
    B, T, H, N = r.shape
    return tuple(torch.empty_like(r) for _ in range(6)) + (r.new_empty((B, H, N, N), dtype=torch.float32),)


def _fwd_setup_context(ctx, inputs, output):
    r, w, k, v, a, b, h0, want_state, state_map = inputs
    ctx.save_for_backward(r, w, k, v, a, b, h0, state_map)   # inputs only: the backward recomputes
    ctx.want_state = want_state


def _fwd_backward(ctx, d_o, d_ht):
    r, w, k, v, a, b, h0_arg, state_map = ctx.saved_tensors
    # with a map the backward kernels see the gathered states; dh0 is scattered back below.  The map is clamped
    # as the kernels clamp it: a map that came on the device was never checked (no read-back), and an entry out
    # of range must not trip a device-side assertion here either
    rows = None if state_map is None else state_map.long().clamp_(0, h0_arg.shape[0] - 1)
    h0 = h0_arg if rows is None else h0_arg.index_select(0, rows)
    dt = r.dtype
    d_ht_c = None
    if ctx.want_state and d_ht is not None and d_ht.numel() > 0:
        d_ht_c = d_ht.to(torch.float32).contiguous()
    if dt == torch.float32 and r.shape[-1] == HEAD_SIZE:
        # float32 calls get float32 gradients: the chunked float32 backward (a dozen tokens or fewer: the recurrent one)
        d_o_c = None if d_o is None else d_o.to(dt).contiguous()
        dr, dw, dk, dv, da, db, dh0 = torch.ops.rwkv_ops_amd.rwkv7_bwd(r, w, k, v, a, b, h0, d_o_c, d_ht_c)
    elif r.shape[-1] != HEAD_SIZE:
        # head size 128 has no chunked backward: the float32 recurrent backward, which reads any of the three
        # dtypes as it is
        d_o_c = None if d_o is None else d_o.to(dt).contiguous()
        dr, dw, dk, dv, da, db, dh0 = torch.ops.rwkv_ops_amd.rwkv7_bwd_recurrent(
            r, w, k, v, a, b, h0, d_o_c, d_ht_c)
    else:
        # The chunked backward kernels are bf16; float16 inputs are rounded to bf16 for them, as the reference's
        # kernel path rounds every input (torch_op.py:451-455).
        cast = (lambda t: t.to(torch.bfloat16)) if dt != torch.bfloat16 else (lambda t: t)
        d_o_c = None if d_o is None else cast(d_o).contiguous()
        dr, dw, dk, dv, da, db, dh0 = torch.ops.rwkv_ops_amd.rwkv7_bwd(
            cast(r), cast(w), cast(k), cast(v), cast(a), cast(b), h0, d_o_c, d_ht_c)
    g0 = None
    if h0 is not None and ctx.needs_input_grad[6]:
        if state_map is not None:
            g0 = torch.zeros_like(h0_arg).index_add_(0, rows, dh0)
        else:
            g0 = dh0.sum(0, keepdim=True) if h0.shape[0] != dh0.shape[0] else dh0
    return dr.to(dt), dw.to(dt), dk.to(dt), dv.to(dt), da.to(dt), db.to(dt), g0, None, None


rwkv7_fwd.register_autograd(_fwd_backward, setup_context=_fwd_setup_context)


# ---- packed sequences (cu_seqlens)
def _fwd_varlen_impl(r, w, k, v, a, b, h0, want_state, cu):
    lib = _lib.load()
    _lib.raise_if_gave_up()
    _, T, H, N = r.shape
    n_seq = cu.numel() - 1
    o = torch.empty_like(r)
    ht = torch.empty((n_seq, H, N, N) if want_state else (0,), dtype=torch.float32, device=r.device)
    code = _dtype_code(r.dtype)
    with _on_device(r.device):
        ws_bytes = lib.rwkv7_fwd_varlen_workspace_bytes(n_seq, T, H, code)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=r.device) if ws_bytes else None
        rc = lib.rwkv7_fwd_varlen(_ptr(r), _ptr(w), _ptr(k), _ptr(v), _ptr(a), _ptr(b), _ptr(cu), n_seq,
                                  _ptr(h0), _h0_stride(h0, n_seq, H), _ptr(o), _ptr(ht) if want_state else None,
                                  T, H, N, N, code, _ptr(ws), ws_bytes, _stream_ptr(r.device))
    _lib.check(rc, "rwkv7_fwd_varlen")
    return o, ht


@torch.library.custom_op("rwkv_ops_amd::rwkv7_fwd_varlen", mutates_args=(), device_types="cuda")
def rwkv7_fwd_varlen(r: torch.Tensor, w: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                     a: torch.Tensor, b: torch.Tensor, h0: Optional[torch.Tensor],
                     want_state: bool, cu: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Inputs ``[1, T, H, 64]`` contiguous, one dtype; ``cu`` int32 ``[n_seq + 1]`` on the device;
    ``h0`` float32 ``[n_seq, H, 64, 64]`` or None.  Returns ``(o, ht)`` with ``ht [n_seq, H, 64, 64]``
    (empty when ``want_state`` is false)."""
    return _fwd_varlen_impl(r, w, k, v, a, b, h0, want_state, cu)


@rwkv7_fwd_varlen.register_fake
def _(r, w, k, v, a, b, h0, want_state, cu):
    _, T, H, N = r.shape
    return torch.empty_like(r), r.new_empty((cu.numel() - 1, H, N, N) if want_state else (0,), dtype=torch.float32)


@torch.library.custom_op("rwkv_ops_amd::rwkv7_bwd_varlen", mutates_args=(), device_types="cuda")
def rwkv7_bwd_varlen(r: torch.Tensor, w: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                     a: torch.Tensor, b: torch.Tensor, h0: Optional[torch.Tensor],
                     d_o: Optional[torch.Tensor], d_ht: Optional[torch.Tensor], cu: torch.Tensor
                     ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor,
                                torch.Tensor, torch.Tensor]:
    """Gradients of ``rwkv7_fwd_varlen`` (bf16 or float32): ``(dr, dw, dk, dv, da, db, dh0)``, ``dh0`` float32
    ``[n_seq, H, 64, 64]``.  Rows of the packed batch that belong to no sequence get zero gradients."""
    lib = _lib.load()
    _, T, H, N = r.shape
    n_seq = cu.numel() - 1
    code = _dtype_code(r.dtype)
    grads = [torch.empty_like(r) for _ in range(6)]
    dh0 = torch.empty((n_seq, H, N, N), dtype=torch.float32, device=r.device)
    with _on_device(r.device):
        ws_bytes = lib.rwkv7_bwd_varlen_workspace_bytes(n_seq, T, H, code)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=r.device)
        rc = lib.rwkv7_bwd_varlen(_ptr(r), _ptr(w), _ptr(k), _ptr(v), _ptr(a), _ptr(b), _ptr(cu), n_seq,
                                  _ptr(h0), _h0_stride(h0, n_seq, H), _ptr(d_o), _ptr(d_ht),
                                  *[_ptr(x) for x in grads], _ptr(dh0),
                                  T, H, N, N, code, _ptr(ws), ws_bytes, _stream_ptr(r.device))
    _lib.check(rc, "rwkv7_bwd_varlen")
    return (*grads, dh0)


@rwkv7_bwd_varlen.register_fake
def _(r, w, k, v, a, b, h0, d_o, d_ht, cu):
    _, T, H, N = r.shape
    return tuple(torch.empty_like(r) for _ in range(6)) + (
        r.new_empty((cu.numel() - 1, H, N, N), dtype=torch.float32),)


@torch.library.custom_op("rwkv_ops_amd::rwkv7_bwd_recurrent_varlen", mutates_args=(), device_types="cuda")
def rwkv7_bwd_recurrent_varlen(r: torch.Tensor, w: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                               a: torch.Tensor, b: torch.Tensor, h0: Optional[torch.Tensor],
                               d_o: Optional[torch.Tensor], d_ht: Optional[torch.Tensor], cu: torch.Tensor
                               ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor,
                                          torch.Tensor, torch.Tensor]:
    """Gradients of ``rwkv7_fwd_varlen`` from the float32 recurrent backward: any of the three dtypes, head size 64
    or 128 (what packed rows at head size 128 get); same arguments and results as ``rwkv7_bwd_varlen``."""
    lib = _lib.load()
    _, T, H, N = r.shape
    n_seq = cu.numel() - 1
    grads = [torch.empty_like(r) for _ in range(6)]
    dh0 = torch.empty((n_seq, H, N, N), dtype=torch.float32, device=r.device)
    with _on_device(r.device):
        ws_bytes = lib.rwkv7_bwd_recurrent_varlen_workspace_bytes(n_seq, T, H, N)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=r.device)
        rc = lib.rwkv7_bwd_recurrent_varlen(_ptr(r), _ptr(w), _ptr(k), _ptr(v), _ptr(a), _ptr(b), _ptr(cu), n_seq,
                                            _ptr(h0), _h0_stride(h0, n_seq, H), _ptr(d_o), _ptr(d_ht),
                                            *[_ptr(x) for x in grads], _ptr(dh0),
                                            T, H, N, N, _dtype_code(r.dtype), _ptr(ws), ws_bytes, _stream_ptr(r.device))
    _lib.check(rc, "rwkv7_bwd_recurrent_varlen")
    return (*grads, dh0)


@rwkv7_bwd_recurrent_varlen.register_fake
def _(r, w, k, v, a, b, h0, d_o, d_ht, cu):
    _, T, H, N = r.shape
    return tuple(torch.empty_like(r) for _ in range(6)) + (
        r.new_empty((cu.numel() - 1, H, N, N), dtype=torch.float32),)


def _fwd_varlen_setup_context(ctx, inputs, output):
    r, w, k, v, a, b, h0, want_state, cu = inputs
    ctx.save_for_backward(r, w, k, v, a, b, h0, cu)
    ctx.want_state = want_state


def _fwd_varlen_backward(ctx, d_o, d_ht):
    r, w, k, v, a, b, h0, cu = ctx.saved_tensors
    dt = r.dtype
    # float32 rows at head size 64 keep float32 (the chunked float32 backward); float16 rows are rounded to bf16 as in
    # the dense call
    d_ht_c = None
    if ctx.want_state and d_ht is not None and d_ht.numel() > 0:
        d_ht_c = d_ht.to(torch.float32).contiguous()
    if r.shape[-1] != HEAD_SIZE:
        # head size 128 has no chunked backward: the float32 recurrent backward, which reads any of the three dtypes
        d_o_c = None if d_o is None else d_o.to(dt).contiguous()
        dr, dw, dk, dv, da, db, dh0 = torch.ops.rwkv_ops_amd.rwkv7_bwd_recurrent_varlen(
            r, w, k, v, a, b, h0, d_o_c, d_ht_c, cu)
        g0 = dh0 if (h0 is not None and ctx.needs_input_grad[6]) else None
        return dr, dw, dk, dv, da, db, g0, None, None
    exact = dt == torch.bfloat16 or dt == torch.float32
    cast = (lambda t: t) if exact else (lambda t: t.to(torch.bfloat16))
    d_o_c = None if d_o is None else cast(d_o.to(dt)).contiguous()
    dr, dw, dk, dv, da, db, dh0 = torch.ops.rwkv_ops_amd.rwkv7_bwd_varlen(
        cast(r), cast(w), cast(k), cast(v), cast(a), cast(b), h0, d_o_c, d_ht_c, cu)
    g0 = dh0 if (h0 is not None and ctx.needs_input_grad[6]) else None
    return dr.to(dt), dw.to(dt), dk.to(dt), dv.to(dt), da.to(dt), db.to(dt), g0, None, None


rwkv7_fwd_varlen.register_autograd(_fwd_varlen_backward, setup_context=_fwd_varlen_setup_context)


@torch.library.custom_op("rwkv_ops_amd::rwkv7_fwd_recurrent", mutates_args=(), device_types="cuda")
def rwkv7_fwd_recurrent(r: torch.Tensor, w: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                        a: torch.Tensor, b: torch.Tensor, h0: Optional[torch.Tensor],
                        want_state: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """The float32 recurrent kernel, same contract as ``rwkv7_fwd``."""
    lib = _lib.load()
    B, T, H, N = r.shape
    o = torch.empty_like(r)
    ht = torch.empty((B, H, N, N) if want_state else (0,), dtype=torch.float32, device=r.device)
    with _on_device(r.device):
        rc = lib.rwkv7_fwd_recurrent(_ptr(r), _ptr(w), _ptr(k), _ptr(v), _ptr(a), _ptr(b),
                                     _ptr(h0), _h0_stride(h0, B, H), _ptr(o),
                                     _ptr(ht) if want_state else None,
                                     B, T, H, N, N, _dtype_code(r.dtype), _stream_ptr(r.device))
    _lib.check(rc, "rwkv7_fwd_recurrent")
    return o, ht


@rwkv7_fwd_recurrent.register_fake
def _(r, w, k, v, a, b, h0, want_state):
    B, T, H, N = r.shape
    return torch.empty_like(r), r.new_empty((B, H, N, N) if want_state else (0,), dtype=torch.float32)


def _decode_impl(r, w, k, v, a, b, state):
    lib = _lib.load()
    B, H, N = r.shape
    o = torch.empty_like(r)
    with _on_device(r.device):
        rc = lib.rwkv7_decode_step(_ptr(r), _ptr(w), _ptr(k), _ptr(v), _ptr(a), _ptr(b),
                                   _ptr(state), H * N * N, _ptr(o), _ptr(state),
                                   B, H, N, N, _dtype_code(r.dtype), _stream_ptr(r.device))
    _lib.check(rc, "rwkv7_decode_step")
    return o


@torch.library.custom_op("rwkv_ops_amd::rwkv7_decode", mutates_args=("state",), device_types="cuda")
def rwkv7_decode(r: torch.Tensor, w: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                 a: torch.Tensor, b: torch.Tensor, state: torch.Tensor) -> torch.Tensor:
    """One token: inputs ``[B, H, 64]``; ``state`` float32 ``[B, H, 64, 64]`` is updated in place."""
    return _decode_impl(r, w, k, v, a, b, state)


@rwkv7_decode.register_fake
def _(r, w, k, v, a, b, state):
    return torch.empty_like(r)


def _decode_pool_impl(r, w, k, v, a, b, states, state_map):
    lib = _lib.load()
    B, H, N = r.shape
    o = torch.empty_like(r)
    with _on_device(r.device):
        rc = lib.rwkv7_decode_step_gather(_ptr(r), _ptr(w), _ptr(k), _ptr(v), _ptr(a), _ptr(b),
                                          _ptr(states), states.shape[0], _ptr(state_map), _ptr(o), None,
                                          B, H, N, N, _dtype_code(r.dtype), _stream_ptr(r.device))
    _lib.check(rc, "rwkv7_decode_step_gather")
    return o


@torch.library.custom_op("rwkv_ops_amd::rwkv7_decode_pool", mutates_args=("states",), device_types="cuda")
def rwkv7_decode_pool(r: torch.Tensor, w: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                      a: torch.Tensor, b: torch.Tensor, states: torch.Tensor,
                      state_map: torch.Tensor) -> torch.Tensor:
    """One token with a pool of states: inputs ``[B, H, 64]``; row b reads and updates in place
    ``states[state_map[b]]`` (float32 ``[n_state, H, 64, 64]``, ``state_map`` int32 ``[B]``, distinct)."""
    return _decode_pool_impl(r, w, k, v, a, b, states, state_map)


@rwkv7_decode_pool.register_fake
def _(r, w, k, v, a, b, states, state_map):
    return torch.empty_like(r)


# --------------------------------------------------------------------------- host logic
HALF_NATIVE_MAX_T = 12     # float16 sequences up to here go to the kernels as they are (the library's RECURRENT_MAX_T)


def _compute_dtype(r: torch.Tensor, T: int = 0) -> torch.dtype:
    # float32 (and float64) inputs take the float32 kernels; everything else is computed
    # from bfloat16 operands, as the reference's kernel path does (torch_op.py:454) -- except
    # float16 decode steps and very short sequences (T given and <= HALF_NATIVE_MAX_T): the decode
    # and recurrent kernels read float16 directly, which saves six cast kernels per step and
    # keeps the three mantissa bits the cast would drop.
    if r.dtype in (torch.float32, torch.float64):
        return torch.float32
    if r.dtype == torch.float16 and 1 <= T <= HALF_NATIVE_MAX_T:
        return torch.float16
    return torch.bfloat16


def _out_dtype(r: torch.Tensor) -> torch.dtype:
    """The dtype of ``out``, whatever the sequence length: float32 for float32 / float64 inputs, float16 for
    float16 inputs (computed from bfloat16 operands beyond HALF_NATIVE_MAX_T tokens and rounded back),
    bfloat16 for everything else."""
    if r.dtype in (torch.float32, torch.float64):
        return torch.float32
    return torch.float16 if r.dtype == torch.float16 else torch.bfloat16


def _prepare(x: torch.Tensor, dtype: torch.dtype, head_first: bool) -> torch.Tensor:
    if head_first:                                   # [B, H, T, K] -> [B, T, H, K]
        x = x.permute(0, 2, 1, 3)
    if x.dtype == dtype and x.is_contiguous():
        return x
    return x.to(dtype).contiguous()


def _as_state_map(state_map, B: int, n_state: int, device: torch.device, distinct: bool = False) -> torch.Tensor:
    """int32 ``[B]`` on ``device``.  A list or a CPU tensor is checked (entries in ``[0, n_state)``, as the
    reference's RWKV6 operator checks its state_map, torch_rwkv_kernel.py:293-297; ``distinct``: no entry
    twice).  A tensor already on the device is taken as it is: reading it back would stall the stream on every
    decode step and cannot happen under graph capture; the kernels clamp what they read, so a bad entry cannot
    fault, and distinct entries are then the caller's contract."""
    if isinstance(state_map, (list, tuple)):
        state_map = torch.tensor(state_map, dtype=torch.int32)
    if not isinstance(state_map, torch.Tensor) or state_map.dtype not in (torch.int32, torch.int64):
        raise ValueError("state_map must be a list or an int32/int64 tensor of shape [B]")
    if tuple(state_map.shape) != (B,):
        raise ValueError(f"state_map must have shape [{B}], got {tuple(state_map.shape)}")
    if not state_map.is_cuda:
        m = state_map.tolist()
        if any(e < 0 or e >= n_state for e in m):
            raise ValueError(f"state_map entries must lie in [0, {n_state})")
        if distinct and len(set(m)) != B:
            raise ValueError("state_map entries must be distinct for an in-place update")
    if state_map.device == device and state_map.dtype == torch.int32 and state_map.is_contiguous():
        return state_map
    return state_map.to(device=device, dtype=torch.int32).contiguous()


def _as_cu_seqlens(cu_seqlens, T: int, device: torch.device) -> torch.Tensor:
    """int32 ``[n_seq + 1]`` on ``device``.  A list or a CPU tensor is checked (starts at 0, never
    decreases, ends at T at most); a tensor already on the device is taken as it is -- reading it back
    would stall the stream, and the kernels clamp what they read, so bad values cannot fault."""
    if isinstance(cu_seqlens, (list, tuple)):
        cu_seqlens = torch.tensor(cu_seqlens, dtype=torch.int32)
    if not isinstance(cu_seqlens, torch.Tensor) or cu_seqlens.dtype not in (torch.int32, torch.int64):
        raise ValueError("cu_seqlens must be a list or an int32/int64 tensor of shape [N + 1]")
    if cu_seqlens.dim() != 1 or cu_seqlens.numel() < 2:
        raise ValueError(f"cu_seqlens must have shape [N + 1] with N >= 1, got {tuple(cu_seqlens.shape)}")
    if not cu_seqlens.is_cuda:
        c = cu_seqlens.tolist()
        if c[0] != 0 or any(y < x for x, y in zip(c, c[1:])) or c[-1] > T:
            raise ValueError(f"cu_seqlens must start at 0, never decrease and end at T = {T} at most, got {c}")
    return cu_seqlens.to(device=device, dtype=torch.int32).contiguous()



def _check_inputs(r, w, k, v, a, b, initial_state, head_first, mapped=False):
    for name, x in zip("rwkvab", (r, w, k, v, a, b)):
        if x.dim() != 4:
            raise ValueError(f"{name} must be 4-D [B, T, H, K] (or [B, H, T, K] with head_first), got {tuple(x.shape)}")
        if x.shape != r.shape:
            raise ValueError(f"{name} has shape {tuple(x.shape)}, expected {tuple(r.shape)} like r")
    for x in (r, w, k, v, a, b):
        _require_gpu(x)
        if x.device != r.device:
            raise ValueError("all inputs must be on one device")
    N = r.shape[-1]
    if N not in HEAD_SIZES:
        raise ValueError(f"head size {N} is not built; only K = V in {HEAD_SIZES}")
    B = r.shape[0]
    H = r.shape[1] if head_first else r.shape[2]
    if min(r.shape) < 1:
        raise ValueError(f"empty input {tuple(r.shape)}")
    if initial_state is not None:
        _require_gpu(initial_state)
        if initial_state.dim() != 4 or tuple(initial_state.shape[1:]) != (H, N, N) \
                or (not mapped and initial_state.shape[0] not in (1, B)) or initial_state.shape[0] < 1:
            raise ValueError(
                f"initial_state must be [N, H, K, V] = [{B} or 1, {H}, {N}, {N}], "
                f"got {tuple(initial_state.shape)}")


def generalized_delta_rule(
    r: torch.Tensor,
    w: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    a: torch.Tensor,
    b: torch.Tensor,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = True,
    head_first: bool = False,
    state_map=None,
    cu_seqlens=None,
):
    """RWKV7 generalized delta rule on MI355X; signature of torch_op.py:458-468 plus ``state_map``.

    ``out`` has the dtype of the inputs for bfloat16, float16 and float32 inputs, whatever T is (the
    reference's kernel path returns bfloat16 for all of them, torch_op.py:451-455,486); float16 sequences of
    more than 12 tokens are computed from bfloat16-rounded operands, as the reference does, and ``out`` is
    rounded back to float16 (an output beyond float16's range, 65504, becomes inf there).  The final state is
    float32 for every input dtype (the reference casts it to the input dtype, torch_op.py:487-488): a decode loop
    can feed it back without loss.

    ``w`` is the raw decay argument: the per-step decay is ``exp(-exp(w))``
    (torch_op.py:433-434), so padded positions use ``w += (1 - mask) * -1e9`` together
    with zeroed r, k, v, a, b (/root/reference/README.md:89-98).

    ``state_map`` (optional, list or int tensor ``[B]``): batch row b starts from
    ``initial_state[state_map[b]]``; ``initial_state`` is then ``[n_state, H, K, V]`` with any
    ``n_state >= 1``.  The final state is always dense ``[B, H, K, V]``.

    ``cu_seqlens`` (optional, list or int tensor ``[N + 1]``, the FlashAttention convention the
    reference's ``chunk_dplr_delta_rule`` documents, torch_op.py:363-365): the inputs are ONE batch row
    ``[1, T, H, K]`` holding N sequences, sequence i = tokens ``cu_seqlens[i] .. cu_seqlens[i+1] - 1``;
    ``initial_state`` and the final state are ``[N, H, K, V]``.  Errors as the reference raises them
    (torch_op.py:388-398); ``head_first`` is not supported with it (torch_op.py:366-368).
    """
    if cu_seqlens is not None:
        return _generalized_delta_rule_varlen(r, w, k, v, a, b, initial_state, output_final_state,
                                              head_first, state_map, cu_seqlens)
    if state_map is not None and initial_state is None:
        raise ValueError("state_map needs an initial_state to index")
    _check_inputs(r, w, k, v, a, b, initial_state, head_first, mapped=state_map is not None)
    dt = _compute_dtype(r, r.shape[2] if head_first else r.shape[1])
    r_, w_, k_, v_, a_, b_ = (_prepare(x, dt, head_first) for x in (r, w, k, v, a, b))
    h0 = None
    if initial_state is not None:
        h0 = initial_state.to(torch.float32).contiguous()
    smap = None
    if state_map is not None:
        smap = _as_state_map(state_map, r_.shape[0], h0.shape[0], r_.device)
    if _direct(r_, w_, k_, v_, a_, b_, h0):
        out, state = _fwd_impl(r_, w_, k_, v_, a_, b_, h0, bool(output_final_state), smap)
    else:
        out, state = torch.ops.rwkv_ops_amd.rwkv7_fwd(r_, w_, k_, v_, a_, b_, h0, bool(output_final_state), smap)
    if out.dtype != _out_dtype(r):
        out = out.to(_out_dtype(r))
    if head_first:
        out = out.permute(0, 2, 1, 3)
    if output_final_state:
        return out, state
    return out


def _generalized_delta_rule_varlen(r, w, k, v, a, b, initial_state, output_final_state, head_first,
                                   state_map, cu_seqlens):
    if head_first:
        raise ValueError("head_first is not supported for variable-length inputs (cu_seqlens)")
    if state_map is not None:
        raise ValueError("state_map and cu_seqlens cannot be combined")
    n_seq = len(cu_seqlens) - 1
    if r.dim() == 4 and r.shape[0] != 1:
        raise ValueError(
            f"The batch size is expected to be 1 rather than {r.shape[0]} when using `cu_seqlens`."
            f"Please flatten variable-length inputs before processing.")
    if initial_state is not None and initial_state.dim() == 4 and initial_state.shape[0] != n_seq:
        raise ValueError(
            f"The number of initial states is expected to be equal to the number of input sequences, "
            f"i.e., {n_seq} rather than {initial_state.shape[0]}.")
    _check_inputs(r, w, k, v, a, b, initial_state, False, mapped=True)
    dt = _compute_dtype(r)
    r_, w_, k_, v_, a_, b_ = (_prepare(x, dt, False) for x in (r, w, k, v, a, b))
    cu = _as_cu_seqlens(cu_seqlens, r_.shape[1], r_.device)
    h0 = None if initial_state is None else initial_state.to(torch.float32).contiguous()
    if _direct(r_, w_, k_, v_, a_, b_, h0):
        out, state = _fwd_varlen_impl(r_, w_, k_, v_, a_, b_, h0, bool(output_final_state), cu)
    else:
        out, state = torch.ops.rwkv_ops_amd.rwkv7_fwd_varlen(r_, w_, k_, v_, a_, b_, h0,
                                                             bool(output_final_state), cu)
    if out.dtype != _out_dtype(r):
        out = out.to(_out_dtype(r))
    if output_final_state:
        return out, state
    return out


def rwkv7_decode_step(r, w, k, v, a, b, state, state_map=None):
    """One decode step with the float32 ``state [B, H, 64, 64]`` updated IN PLACE.

    ``r .. b`` are ``[B, H, 64]`` (or ``[B, 1, H, 64]``); returns ``o`` of the same shape.
    Equivalent to ``generalized_delta_rule`` with T = 1 and ``initial_state=state``, without
    allocating a second state.  With ``state_map`` (list or int tensor ``[B]``, distinct entries)
    ``state`` is a pool ``[n_state, H, 64, 64]`` and row b reads and updates ``state[state_map[b]]``:
    the serving loop's slot table, no gather or scatter of states around the step.  A map given as a list
    or a CPU tensor is checked; an int32 tensor on the device is used as it is, without any read-back, so
    the step never synchronises and can be captured into a graph."""
    squeeze = r.dim() == 4
    xs = [x[:, 0] if squeeze else x for x in (r, w, k, v, a, b)]
    for x in xs:
        _require_gpu(x)
    _require_gpu(state)
    if state.dtype != torch.float32 or not state.is_contiguous():
        raise ValueError("state must be a contiguous float32 tensor [B, H, 64, 64]")
    B, H, N = xs[0].shape
    if state_map is not None:
        if N not in HEAD_SIZES or state.dim() != 4 or tuple(state.shape[1:]) != (H, N, N):
            raise ValueError(f"state must be [n_state, {H}, {N}, {N}] with a head size in {HEAD_SIZES}, got {tuple(state.shape)}")
        smap = _as_state_map(state_map, B, state.shape[0], state.device, distinct=True)
    elif N not in HEAD_SIZES or tuple(state.shape) != (B, H, N, N):
        raise ValueError(f"state must be [{B}, {H}, {N}, {N}] with a head size in {HEAD_SIZES}, got {tuple(state.shape)}")
    dt = _compute_dtype(xs[0], 1)
    xs = [x if (x.dtype == dt and x.is_contiguous()) else x.to(dt).contiguous() for x in xs]
    direct = _direct(*xs, state)
    if state_map is not None:
        o = _decode_pool_impl(*xs, state, smap) if direct else torch.ops.rwkv_ops_amd.rwkv7_decode_pool(*xs, state, smap)
    else:
        o = _decode_impl(*xs, state) if direct else torch.ops.rwkv_ops_amd.rwkv7_decode(*xs, state)
    return o[:, None] if squeeze else o
