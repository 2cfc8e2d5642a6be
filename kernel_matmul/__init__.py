"""Drop-in alias: ``import kernel_matmul...`` resolves to the MI355X implementation.

Code written against Turakar/kernel-matmul imports ``kernel_matmul.native_function``,
``kernel_matmul.ranges``, ``kernel_matmul.linear_operator`` and so on.  A meta path finder
binds every ``kernel_matmul.<name>`` to the very module object ``kernel_matmul_amd.<name>``
(not a copy), so module-level state such as the active compile pool is shared.
"""
import importlib
import importlib.abc
import importlib.util
import sys

from kernel_matmul_amd import _BLOCK_SIZE, __version__  # noqa: F401

_PREFIX = __name__ + "."
_TARGET = "kernel_matmul_amd."


class _AliasFinder(importlib.abc.MetaPathFinder, importlib.abc.Loader):
    def find_spec(self, fullname, path=None, target=None):
        if not fullname.startswith(_PREFIX):
            return None
        real = _TARGET + fullname[len(_PREFIX):]
        if importlib.util.find_spec(real) is None:
            return None
        return importlib.util.spec_from_loader(fullname, self)

    def create_module(self, spec):
        module = importlib.import_module(_TARGET + spec.name[len(_PREFIX):])
        self._real_spec = module.__spec__
        return module

    def exec_module(self, module):
        module.__spec__ = self._real_spec  # the import system replaced it with the alias spec


sys.meta_path.insert(0, _AliasFinder())
