"""``pla.prefill.flashkdapro`` drop-in (pla/prefill/flashkdapro/__init__.py)."""
from .ops import flashkda_fwd, CHUNK_SIZE  # noqa: F401

__all__ = ["flashkda_fwd"]
