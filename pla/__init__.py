"""``pla``: the reference's import path for the MI355X implementation.

Code written against the reference imports ``pla.decode``, ``pla.decode.kda``, ``pla.decode.private``,
``pla.decode.kda_replayssm_sglang`` / ``kda_mtp_sglang``, ``pla.decode.kda_replayssm_vllm``,
``pla.prefill.flashqla`` and ``pla.prefill.flashkdapro`` (pla/__init__.py:31-53 of the reference; nothing is
exported from the root).  Here every ``pla.X`` is the module object ``pla_amd.X``: a finder on
``sys.meta_path`` resolves any name under ``pla.`` by importing its ``pla_amd.`` counterpart and registering that
one module under both names, so the two spellings share state (caches, the loaded library) and
``pla.decode._C`` is the compiled extension ``pla_amd.decode._C``.
"""

import importlib
import importlib.abc
import importlib.util
import sys

import pla_amd

__version__ = pla_amd.__version__
__all__ = []


class _AliasLoader(importlib.abc.Loader):
    """Hands importlib the pla_amd module itself.  importlib then stamps the alias spec (and loader) on whatever
    module a loader returns; ``exec_module`` puts the module's own ones back, so that ``pla_amd.X`` keeps
    ``__spec__.name == "pla_amd.X"`` (relative imports inside it, ``importlib.reload`` and ``pkgutil`` go on
    using the real spec) while ``sys.modules["pla.X"]`` is the same object."""

    def __init__(self, target):
        self._target = target
        self._own = None

    def create_module(self, spec):
        module = importlib.import_module(self._target)    # the pla_amd module itself, not a copy
        self._own = (module.__spec__, getattr(module, "__loader__", None))
        return module

    def exec_module(self, module):
        if self._own is not None:
            module.__spec__, module.__loader__ = self._own


class _AliasFinder(importlib.abc.MetaPathFinder):
    def find_spec(self, fullname, path=None, target=None):
        if not fullname.startswith("pla."):
            return None
        real = "pla_amd." + fullname[len("pla."):]
        try:
            found = importlib.util.find_spec(real)
        except ModuleNotFoundError:
            return None
        if found is None:
            return None
        spec = importlib.util.spec_from_loader(fullname, _AliasLoader(real), is_package=found.submodule_search_locations is not None)
        return spec


if not any(isinstance(f, _AliasFinder) for f in sys.meta_path):
    sys.meta_path.insert(0, _AliasFinder())


def __getattr__(name):
    if name in ("decode", "prefill"):
        return importlib.import_module("pla." + name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
