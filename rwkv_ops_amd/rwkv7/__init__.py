from .op import generalized_delta_rule, rwkv7_decode_step, last_forward_status, HEAD_SIZE  # noqa: F401
from .resets import cu_seqlens_from_resets, generalized_delta_rule_resets  # noqa: F401
