"""Padded batches with per-row lengths and in-row state resets, on the packed-sequence kernels.

The reference's XLA-FFI kernel for RWKV7 takes, next to a padded batch ``[B, T, H, K]``, a ``length`` per
batch row and a boolean ``new_starts`` per token
(/root/reference/rwkv_ops/rwkv7_kernel/cuda_kernel/wkv7_jax.cu:18,23-24,46-51,66): the state is set to
zero before every token whose ``new_starts`` flag is set (several documents in one row), and the state
handed back is the one after token ``length - 1`` (rows padded at the end).  Its torch operator has no
such arguments.  Both mean "this row is several independent sequences", which is what ``cu_seqlens``
says, so the function here builds that table and calls ``generalized_delta_rule`` once on the batch
viewed as one packed row -- no copy of the inputs, no kernel of its own.

What differs from the reference's kernel, deliberately: outputs at the padded positions (``t >= length``)
are those of a sequence that starts from a zero state there, where the reference keeps running the row's
state (both are padding that no caller reads); a row of length 0 hands back the state it started from
(the reference leaves that value unset).
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from .op import generalized_delta_rule

__all__ = ["cu_seqlens_from_resets", "generalized_delta_rule_resets"]


def _as_host_list(x, name: str):
    if x is None:
        return None
    if isinstance(x, torch.Tensor):
        return x.detach().cpu().tolist()          # (a device tensor is read back: this helper is host logic)
    return [list(row) if isinstance(row, (list, tuple)) else row for row in x]


def cu_seqlens_from_resets(B: int, T: int, length=None, new_starts=None) -> Tuple[List[int], List[int], List[int]]:
    """The packed-sequence table of a ``[B, T]`` batch flattened to one row of ``B * T`` tokens.

    Returns ``(cu_seqlens, first, last)``: ``first[b]`` is the index of the sequence that starts at row b's
    first token and takes the row's initial state (-1 when ``new_starts[b][0]`` is set: the row starts from
    zero), ``last[b]`` the index of the sequence whose final state is the row's (the one that ends at token
    ``length[b]``; -1 for a row of length 0)."""
    length = _as_host_list(length, "length")
    new_starts = _as_host_list(new_starts, "new_starts")
    if length is None:
        length = [T] * B
    if len(length) != B or any((not 0 <= int(n) <= T) for n in length):
        raise ValueError(f"length must hold B = {B} values in 0 .. T = {T}")
    if new_starts is not None and (len(new_starts) != B or any(len(row) != T for row in new_starts)):
        raise ValueError(f"new_starts must be [B, T] = [{B}, {T}]")
    cu, first, last = [0], [], []
    for b in range(B):
        n = int(length[b])
        cuts = {0}
        if new_starts is not None:
            cuts.update(t for t in range(1, T) if new_starts[b][t])
        if 0 < n < T:
            cuts.add(n)
        cuts = sorted(cuts)
        reset_at_0 = bool(new_starts is not None and new_starts[b][0])
        first.append(-1 if reset_at_0 else len(cu) - 1)
        last_b = -1
        for i, t0 in enumerate(cuts):
            t1 = cuts[i + 1] if i + 1 < len(cuts) else T
            if t1 == n:
                last_b = len(cu) - 1
            cu.append(b * T + t1)
        last.append(last_b)
    return cu, first, last


def generalized_delta_rule_resets(r, w, k, v, a, b, initial_state: Optional[torch.Tensor] = None,
                                  length=None, new_starts=None, output_final_state: bool = True):
    """``generalized_delta_rule`` on a padded batch ``[B, T, H, K]`` whose rows hold ``length[b]`` valid tokens
    and restart from a zero state wherever ``new_starts[b, t]`` is set.  ``initial_state`` is ``[B, H, K, V]``
    (or ``[1, H, K, V]``, shared); returns ``out [B, T, H, K]`` and, with ``output_final_state``, the state of
    every row after its last valid token, ``[B, H, K, V]`` float32.  Differentiable like the packed call it makes."""
    if r.dim() != 4:
        raise ValueError(f"r must be [B, T, H, K], got {tuple(r.shape)}")
    B, T, H, K = r.shape
    cu, first, last = cu_seqlens_from_resets(B, T, length, new_starts)
    n_seq = len(cu) - 1
    V = v.shape[-1]
    flat = [x.reshape(1, B * T, *x.shape[2:]) for x in (r, w, k, v, a, b)]
    h0 = None
    if initial_state is not None:
        if initial_state.dim() != 4 or initial_state.shape[0] not in (1, B) or tuple(initial_state.shape[1:]) != (H, K, V):
            raise ValueError(f"initial_state must be [{B} or 1, {H}, {K}, {V}], got {tuple(initial_state.shape)}")
        rows = [b_ for b_ in range(B) if first[b_] >= 0]
        h0 = torch.zeros((n_seq, H, K, V), dtype=torch.float32, device=r.device)
        if rows:
            src = initial_state.to(torch.float32)
            src = src.expand(B, -1, -1, -1) if src.shape[0] == 1 else src
            idx = torch.tensor([first[b_] for b_ in rows], device=r.device)
            h0 = h0.index_copy(0, idx, src[torch.tensor(rows, device=r.device)])
    res = generalized_delta_rule(*flat, initial_state=h0, output_final_state=output_final_state, cu_seqlens=cu)
    if not output_final_state:
        return res.reshape(B, T, H, V)
    out, states = res
    pick = torch.tensor([max(j, 0) for j in last], device=r.device)
    final = states.index_select(0, pick)
    empty = [b_ for b_ in range(B) if last[b_] < 0]
    if empty:                                      # no valid token: the state the row started from
        start = torch.zeros((B, H, K, V), dtype=torch.float32, device=r.device)
        if initial_state is not None:
            src = initial_state.to(torch.float32)
            src = src.expand(B, -1, -1, -1) if src.shape[0] == 1 else src
            keep = torch.tensor([1.0 if first[b_] >= 0 else 0.0 for b_ in range(B)], device=r.device)
            start = src * keep.view(B, 1, 1, 1)
        mask = torch.zeros(B, dtype=torch.bool, device=r.device)
        mask[torch.tensor(empty, device=r.device)] = True
        final = torch.where(mask.view(B, 1, 1, 1), start, final)
    return out.reshape(B, T, H, V), final
