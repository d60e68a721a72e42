"""``pla.prefill.flashqla`` drop-in (pla/prefill/flashqla/__init__.py:46-53)."""
from .ops import chunk_gated_delta_rule_fwd, gdn_prefill_packed_qkv_fwd, CHUNK_SIZE  # noqa: F401

__all__ = ["chunk_gated_delta_rule_fwd", "gdn_prefill_packed_qkv_fwd"]
