"""The package under the reference's import name.

The reference's scripts import their engine as ``tinyvllm`` (tinyvllm/__init__.py:1-2 exports ``LLM`` and
``SamplingParams``; bench.py:31 and example.py:2 do ``from tinyvllm import LLM, SamplingParams``), and code
written against it reaches the layers as ``tinyvllm.layers.attention`` and so on.  ``install()`` makes every
such import resolve to THE SAME module objects as ``tinyllmforge_amd...`` (one ``Context``, one set of
classes), so a script of the reference runs against this package with two lines in front of its imports:

    import tinyllmforge_amd.dropin
    tinyllmforge_amd.dropin.install()

A plain ``sys.modules["tinyvllm"] = tinyllmforge_amd`` is not enough: sub-module imports would then load
second copies of the files under the other name, each with its own module globals.
"""
from __future__ import annotations

import importlib
import importlib.abc
import importlib.machinery
import sys

_REAL = __name__.rsplit(".", 1)[0]


class _AliasLoader(importlib.abc.Loader):
    def __init__(self, real_name: str):
        self.real_name = real_name

    def create_module(self, spec):
        return importlib.import_module(self.real_name)

    def exec_module(self, module):      # the real module has run already
        pass


class _AliasFinder(importlib.abc.MetaPathFinder):
    def __init__(self, alias: str):
        self.alias = alias

    def find_spec(self, fullname, path=None, target=None):
        if fullname != self.alias and not fullname.startswith(self.alias + "."):
            return None
        real_name = _REAL + fullname[len(self.alias):]
        try:
            real = importlib.import_module(real_name)
        except ModuleNotFoundError as e:
            if e.name == real_name:
                return None
            raise
        spec = importlib.machinery.ModuleSpec(fullname, _AliasLoader(real_name), is_package=hasattr(real, "__path__"))
        return spec


def install(alias: str = "tinyvllm") -> None:
    """Register ``alias`` (and every ``alias.x.y``) as another name of this package's modules.  The module
    objects keep their own ``__name__`` / ``__spec__``: importing under the alias only looks them up."""
    for f in sys.meta_path:
        if isinstance(f, _AliasFinder) and f.alias == alias:
            return
    if alias in sys.modules and sys.modules[alias] is not sys.modules[_REAL]:
        raise ImportError(f"another module named {alias!r} is already imported")
    sys.meta_path.insert(0, _AliasFinder(alias))
    sys.modules[alias] = sys.modules[_REAL]


def uninstall(alias: str = "tinyvllm") -> None:
    sys.meta_path[:] = [f for f in sys.meta_path if not (isinstance(f, _AliasFinder) and f.alias == alias)]
    for name in [n for n in sys.modules if n == alias or n.startswith(alias + ".")]:
        del sys.modules[name]
