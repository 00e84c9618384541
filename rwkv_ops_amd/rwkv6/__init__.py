"""The RWKV6 operator on MI355X: host side.

Mirrors the operator class of the reference
(/root/reference/rwkv_ops/rwkv6_kernel/__init__.py:37-96, torch_rwkv_kernel.py:10-330,
ops_rwkv_kernel.py:5-83):

    op = RWKVKernelOperator(head_size, max_sequence_length)
    y, state = op(r, k, v, w, u, with_state=False, init_state=None, state_map=None)

``r, k, v, w`` are ``[B, T, C]`` with ``C = H * head_size``, ``u`` is ``[H, head_size]`` (or ``[C]``);
``init_state`` is ``[n_state, H, K, V]`` or ``[H, K, V]``; ``state_map`` (list or int tensor ``[B]``) lets
row b start from ``init_state[state_map[b]]`` and is inferred for ``n_state`` 1 or B
(torch_rwkv_kernel.py:286-313).  Returns ``(y, state)`` with ``with_state`` else ``(y, None)``
(torch_rwkv_kernel.py:326-330); ``y`` has the inputs' dtype (float32 for float16 inputs) and so has the
state (torch_rwkv_kernel.py:166-170,236-239).

Differences, deliberate: an ``init_state`` of any float dtype is accepted (the reference asserts the inputs'
dtype); the state is carried in float32 inside the kernels whatever the inputs are and only rounded to
the inputs' dtype on return; pass ``state_dtype=torch.float32`` to the constructor to get it back
unrounded, which is what a decode loop should feed back.

Gradients: as in the reference, the call without a state is differentiable (torch_rwkv_kernel.py:57-152:
gradients of r, k, v, w and u); with ``with_state`` or an ``init_state`` tensors that require grad raise.
The backward (``rwkv6_bwd``) runs the RWKV7 backward kernels on operands read one token ahead (see
``_Rwkv6Function``) plus an epilogue kernel for the bonus term.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..rwkv7 import _lib
from ..rwkv7.op import _as_state_map, _dtype_code, _on_device, _ptr, _require_gpu, _stream_ptr

__all__ = ["RWKVKernelOperator", "get_rwkv6_kernel"]

HEAD_SIZES = (64, 128)


def _forward(xs, states, n_state, smap, with_state, B, T, H, N, dt):
    """One rwkv6_fwd call: ``xs`` = (r, k, v, w, u) contiguous in ``dt``; returns (y, final states or None)."""
    code = _dtype_code(dt)
    lib = _lib.load()
    dev = xs[0].device
    y = torch.empty((B, T, H * N), dtype=dt, device=dev)
    ys = torch.empty((B, H, N, N), dtype=torch.float32, device=dev) if with_state else None
    with _on_device(dev):
        ws_bytes = lib.rwkv6_fwd_workspace_bytes(B, T, H, code) if N == 64 else 0     # head size 128: no workspace
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
        rc = lib.rwkv6_fwd(*[_ptr(x) for x in xs], _ptr(states), n_state, _ptr(smap), _ptr(y), _ptr(ys),
                           B, T, H, N, N, code, _ptr(ws), ws_bytes, _stream_ptr(dev))
    _lib.check(rc, "rwkv6_fwd")
    return y, ys


class _Rwkv6Function(torch.autograd.Function):
    """The stateless call with gradients.

    With zero a and b the RWKV7 operator keeps RWKV6's state, s_t = diag(d_t) s_{t-1} + k_t v_t^T, and
    outputs o_t = r_t s_t, while RWKV6 outputs y_t = r_t s_{t-1} + (r_t . u * k_t) v_t.  So with r shifted
    by one token, r'_t = r_{t+1}, the RWKV7 output is y without its bonus term, shifted the other way:
    o'_t = y_{t+1} - bonus_{t+1} (and y_0 is all bonus, the initial state being zero).  The backward
    (``rwkv6_bwd`` in the library) therefore is the RWKV7 backward kernels on (r', w, k, v, 0, 0) with the
    upstream gradient read one token ahead like r, its dr moved back, and an epilogue kernel for the bonus
    term and du."""

    @staticmethod
    def forward(ctx, r, k, v, w, u, H):
        B, T, _ = r.shape
        y, _ = _forward((r, k, v, w, u), None, 0, None, False, B, T, H, r.shape[2] // H, r.dtype)
        ctx.save_for_backward(r, k, v, w, u)
        ctx.H = H
        return y

    @staticmethod
    def backward(ctx, gy):
        r, k, v, w, u = ctx.saved_tensors
        B, T, C = r.shape
        H = ctx.H
        N = C // H
        dt = r.dtype                       # bfloat16 or float32: the kernels of that type (float32 gradients for
        code = _dtype_code(dt)             # float32 tensors, torch_rwkv_kernel.py:137)
        g = gy.to(dt).contiguous()
        lib = _lib.load()
        grads = [torch.empty((B, T, C), dtype=dt, device=r.device) for _ in range(4)]
        du = torch.empty((H, N), dtype=torch.float32, device=r.device)
        with _on_device(r.device):
            ws_bytes = lib.rwkv6_bwd_workspace_bytes_head(B, T, H, N, code)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=r.device)
            rc = lib.rwkv6_bwd(*[_ptr(x) for x in (r, k, v, w, u)], _ptr(g), *[_ptr(x) for x in grads], _ptr(du),
                               B, T, H, N, N, code, _ptr(ws), ws_bytes, _stream_ptr(r.device))
        _lib.check(rc, "rwkv6_bwd")
        dr, dk, dv, dw = (x.to(dt) for x in grads)
        return dr, dk, dv, dw, du.reshape(u.shape).to(u.dtype), None


class RWKVKernelOperator:
    def __init__(self, head_size: int, max_sequence_length: Optional[int] = None,
                 state_dtype: Optional[torch.dtype] = None):
        if int(head_size) not in HEAD_SIZES:
            # (the reference compiles its kernels for the head size it is given, torch_rwkv_kernel.py:22-45)
            raise NotImplementedError(f"head_size={head_size}: head sizes {HEAD_SIZES} are built")
        self.head_size = int(head_size)
        self.max_sequence_length = max_sequence_length      # the kernels have no length limit
        self.state_dtype = state_dtype

    def __call__(self, r, k, v, w, u, with_state=False, init_state=None, state_map=None):
        if not isinstance(u, torch.Tensor):
            u = u.value                                      # a keras variable, torch_rwkv_kernel.py:219-220
        for name, x in zip("rkvw", (r, k, v, w)):
            if x.dim() != 3 or x.shape != r.shape:
                raise ValueError(f"{name} must be [B, T, C] like r, got {tuple(x.shape)}")
        B, T, C = r.shape
        if C % self.head_size != 0:
            raise ValueError(f"C = {C} is not a multiple of the head size {self.head_size}")
        H = C // self.head_size
        if u.numel() != C:
            raise ValueError(f"u must have H * head_size = {C} elements, got {tuple(u.shape)}")
        if min(B, T, H) < 1:
            raise ValueError(f"empty input {tuple(r.shape)}")
        if not (r.dtype == k.dtype == v.dtype == w.dtype == u.dtype):
            raise ValueError("r, k, v, w, u must share one dtype")          # torch_rwkv_kernel.py:232
        if r.dtype not in (torch.float32, torch.bfloat16, torch.float16):
            raise ValueError(f"unsupported dtype {r.dtype}")
        for x in (r, k, v, w, u):
            _require_gpu(x)
            if x.device != r.device:
                raise ValueError("all inputs must be on one device")
        needs_grad = torch.is_grad_enabled() and any(x.requires_grad for x in (r, k, v, w, u))
        if needs_grad and (with_state or init_state is not None):
            raise NotImplementedError("gradients are built for the call without a state only, as in the reference "
                                      "(torch_rwkv_kernel.py:57-152); call under torch.no_grad() or drop the state")
        out_dtype = r.dtype if r.dtype != torch.float16 else torch.float32

        states, n_state, smap = None, 0, None
        if init_state is not None:
            if init_state.dim() not in (3, 4):
                raise ValueError("init_state must be [n_state, H, K, V] or [H, K, V]")
            if init_state.dim() == 3:
                init_state = init_state[None]
            if tuple(init_state.shape[1:]) != (H, self.head_size, self.head_size) or init_state.shape[0] > B:
                raise ValueError(f"init_state must be [n_state <= {B}, {H}, {self.head_size}, {self.head_size}], "
                                 f"got {tuple(init_state.shape)}")
            _require_gpu(init_state)
            n_state = init_state.shape[0]
            states = init_state.to(torch.float32).contiguous()
            if state_map is None:
                if n_state not in (1, B):
                    raise ValueError("state_map cannot be inferred: give it explicitly")
            else:
                # a list or a CPU tensor is checked (torch_rwkv_kernel.py:293-297); a tensor on the device is taken
                # as it is, without a read-back that would stall the stream (the kernels clamp what they read)
                smap = _as_state_map(state_map, B, n_state, r.device)
        elif state_map is not None:
            raise ValueError("state_map needs an init_state to index")

        # float16 has no kernel of its own: its values are exact in float32
        dt = torch.bfloat16 if r.dtype == torch.bfloat16 else torch.float32
        xs = [x if (x.dtype == dt and x.is_contiguous()) else x.to(dt).contiguous() for x in (r, k, v, w, u)]
        if needs_grad:
            return _Rwkv6Function.apply(*xs, H).to(out_dtype), None
        y, ys = _forward(xs, states, n_state, smap, with_state, B, T, H, self.head_size, dt)
        y = y.to(out_dtype)
        if not with_state:
            return y, None
        return y, ys.to(self.state_dtype if self.state_dtype is not None else out_dtype)


def get_rwkv6_kernel(KERNEL_TYPE: str = "hip"):
    """The operator class, as /root/reference/rwkv_ops/rwkv6_kernel/__init__.py:9 returns it.  "hip" and,
    for callers written against the reference, "cuda" and "triton" select the MI355X kernels; "native" is
    refused: there is no eager implementation in this package."""
    if str(KERNEL_TYPE).lower() not in ("hip", "cuda", "triton"):
        raise NotImplementedError(f"KERNEL_TYPE={KERNEL_TYPE!r}: rwkv_ops_amd only has the MI355X HIP kernels")
    return RWKVKernelOperator
