"""``import appy`` resolves to :mod:`appy_amd`, so programs written for the
reference package (``import appy`` / ``@appy.jit`` / ``import appy.np_shared``)
run unchanged.  Submodules are the ``appy_amd`` ones under a second name, not
second copies (module-level state such as the device-mirror registry exists
once)."""
import importlib as _importlib
import importlib.abc as _abc
import importlib.machinery as _machinery
import sys as _sys

import appy_amd as _impl


class _Alias(_abc.MetaPathFinder, _abc.Loader):
    def find_spec(self, fullname, path=None, target=None):
        if fullname.startswith("appy."):
            return _machinery.ModuleSpec(fullname, self)
        return None

    def create_module(self, spec):
        return _importlib.import_module("appy_amd" + spec.name[len("appy"):])

    def exec_module(self, module):
        pass


if not any(isinstance(f, _Alias) for f in _sys.meta_path):
    _sys.meta_path.insert(0, _Alias())
_sys.modules[__name__] = _impl
