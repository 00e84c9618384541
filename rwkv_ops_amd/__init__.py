"""rwkv_ops_amd: the RWKV7 generalized delta rule of pass-lin/rwkv_ops, MI355X-native.

Same façade as the reference package (/root/reference/rwkv_ops/__init__.py:22-28):

    from rwkv_ops_amd import generalized_delta_rule, rwkv7_op, RWKV7_USE_KERNEL
    from rwkv_ops_amd import get_generalized_delta_rule
    from rwkv_ops_amd import RWKV6_OP, get_rwkv6_kernel      # the RWKV6 operator class

``get_generalized_delta_rule(HEAD_SIZE=64, KERNEL_TYPE="hip") -> (fn, USE_KERNEL)``
follows /root/reference/rwkv_ops/rwkv7_kernel/__init__.py:14,156.  There is one
implementation, the gfx950 HIP kernels; ``USE_KERNEL`` is therefore always True and
callers use the kernel-path padding recipe (``w += (1 - mask) * -1e9``,
/root/reference/README.md:89-98).
"""
from __future__ import annotations

__version__ = "0.1"

from .rwkv7 import generalized_delta_rule as _hip_generalized_delta_rule
from .rwkv7 import rwkv7_decode_step, last_forward_status  # noqa: F401
from .rwkv7 import generalized_delta_rule_resets  # noqa: F401
from .rwkv6 import get_rwkv6_kernel


def get_generalized_delta_rule(HEAD_SIZE: int = 64, KERNEL_TYPE: str = "hip"):
    """Returns ``(generalized_delta_rule, USE_KERNEL)``.

    ``KERNEL_TYPE`` accepts "hip" and, for callers written against the reference, its
    GPU kernel names "triton" and "cuda": they all select the HIP kernels.  "native" is
    refused: this package ships no CPU or eager implementation.  The function returned takes the head
    size from its arguments: 64 has every kernel; 128 (the head size of the reference's own value test,
    /root/reference/test_script/test_rwkv7_value.py:51) has the decode step, a chunked bf16 forward, and
    token-by-token float32 kernels for everything else, gradients included (no chunked backward)."""
    if int(HEAD_SIZE) not in (64, 128):
        raise NotImplementedError(f"HEAD_SIZE={HEAD_SIZE}: head sizes 64 and 128 are built")
    kt = str(KERNEL_TYPE).lower()
    if kt not in ("hip", "triton", "cuda"):
        raise NotImplementedError(
            f"KERNEL_TYPE={KERNEL_TYPE!r}: rwkv_ops_amd only has the MI355X HIP kernels "
            "('hip'; 'triton' and 'cuda' are accepted as aliases)")
    return _hip_generalized_delta_rule, True


generalized_delta_rule, RWKV7_USE_KERNEL = get_generalized_delta_rule()
rwkv7_op = generalized_delta_rule
RWKV6_OP = get_rwkv6_kernel()                     # /root/reference/rwkv_ops/__init__.py:29
