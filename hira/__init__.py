"""``hira``: the import path the reference installs itself under (setup.py:14-15 maps the
package ``hira`` onto its source tree; its own modules import each other that way, e.g.
searcher/cpu.py:3,6 and cache/hira_cache.py:7-10).

Every ``hira.X`` resolves to the very module object ``hira_amd.X`` — not to a second copy of it —
so ``hira.indexer.CUDAIndexer is hira_amd.indexer.CUDAIndexer`` and a test that patches a name in
``hira.cache.hira_cache`` patches the module the cache layer reads.  The reference's file names
for the GPU backend are kept as well: ``hira.indexer.cuda`` and ``hira.searcher.cuda`` are the
``hip`` modules here (PyTorch-ROCm calls the MI355X "cuda").  Nothing is imported until asked for.
"""
from __future__ import annotations

import importlib
import importlib.abc
import importlib.machinery
import importlib.util
import sys

import hira_amd

__version__ = hira_amd.__version__
__all__ = []

_RENAMED = {"indexer.cuda": "indexer.hip", "searcher.cuda": "searcher.hip"}


class _Alias(importlib.abc.MetaPathFinder, importlib.abc.Loader):
    """Finds ``hira.a.b`` by importing ``hira_amd.a.b`` and handing that module back."""

    def find_spec(self, fullname, path=None, target=None):
        if not fullname.startswith("hira."):
            return None
        rest = fullname[len("hira."):]
        real = "hira_amd." + _RENAMED.get(rest, rest)
        try:
            found = importlib.util.find_spec(real)
        except ModuleNotFoundError:
            found = None
        if found is None:
            return None
        spec = importlib.machinery.ModuleSpec(fullname, self, origin=real,
                                              is_package=found.submodule_search_locations is not None)
        spec.loader_state = real
        return spec

    def create_module(self, spec):
        module = importlib.import_module(spec.loader_state)
        spec.loader_state = module.__spec__
        return module

    def exec_module(self, module):
        # the import system has just pointed the module at the alias's spec: give it its own back
        module.__spec__ = module.__spec__.loader_state


if not any(isinstance(f, _Alias) for f in sys.meta_path):
    sys.meta_path.insert(0, _Alias())
