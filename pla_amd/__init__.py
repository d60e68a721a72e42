"""pla_amd: MI355X (gfx950) implementation of PLA's gated delta-rule path.

Sub-packages mirror the reference's ``pla`` namespace (pla/__init__.py:31-53):
``pla_amd.decode``, ``pla_amd.decode.private``, ``pla_amd.decode.kda``,
``pla_amd.decode.kda_replayssm_sglang`` (also under its former name ``kda_mtp_sglang``),
``pla_amd.decode.kda_replayssm_vllm``, ``pla_amd.prefill.flashqla`` and
``pla_amd.prefill.flashkdapro``.  ``import pla_amd as pla`` is the drop-in.
Sub-packages are imported lazily so that importing the top level never loads
the native library.
"""

import importlib

__version__ = "0.1"
_SUBMODULES = ("decode", "prefill")


def __getattr__(name):
    if name in _SUBMODULES:
        return importlib.import_module("." + name, __name__)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
