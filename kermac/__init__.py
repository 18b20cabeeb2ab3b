"""``import kermac`` -- the reference's module name -- resolves to the MI355X
implementation: ``kermac`` *is* the ``kermac_amd`` module, and ``kermac.<submodule>``
is ``kermac_amd.<submodule>`` (one module object each, so enum members and the
``ModuleCache`` singleton are the same under both names).  Code written against the
reference (``import kermac``; ``kermac.cdist``, ``kermac.run_kernel``,
``kermac.cdist_grad``, ``from kermac.common import tensor_stats`` ...) runs unchanged.
"""
import importlib
import importlib.abc
import importlib.util
import sys

_ALIAS = "kermac"
_REAL = "kermac_amd"


class _AliasFinder(importlib.abc.MetaPathFinder, importlib.abc.Loader):
    """Serves ``kermac.x.y`` with the module object of ``kermac_amd.x.y``."""

    def find_spec(self, fullname, path=None, target=None):
        if fullname.startswith(_ALIAS + "."):
            return importlib.util.spec_from_loader(fullname, self)
        return None

    def create_module(self, spec):
        return importlib.import_module(_REAL + spec.name[len(_ALIAS):])

    def exec_module(self, module):
        pass                      # already executed under its own name


_real = importlib.import_module(_REAL)
if not any(isinstance(finder, _AliasFinder) for finder in sys.meta_path):
    sys.meta_path.insert(0, _AliasFinder())
for _name, _module in list(sys.modules.items()):
    if _name.startswith(_REAL + "."):
        sys.modules[_ALIAS + _name[len(_REAL):]] = _module
sys.modules[_ALIAS] = _real
