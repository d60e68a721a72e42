"""Former name of ``pla_amd.decode.kda_replayssm_sglang`` (the reference keeps the same alias package,
pla/decode/kda_mtp_sglang/__init__.py:33-41): both names give the same functions."""

from ..kda_replayssm_sglang import commit_kda_replayssm_after_verify, fused_kda_decode_mtp_dspark

__all__ = ["fused_kda_decode_mtp_dspark", "commit_kda_replayssm_after_verify"]
