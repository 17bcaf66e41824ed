"""`warpconvnet` import path for code written against the reference package.

Every module of this name resolves to the module of the same relative path in `warpconvnet_amd`
(the same module object, not a copy), so `from warpconvnet.nn.modules.sparse_conv import
SparseConv3d`, `from warpconvnet.geometry.types.voxels import Voxels` and
`from warpconvnet.nn.functional.sparse_conv import spatially_sparse_conv` work unchanged
(the reference's own imports: tests/nn/test_sparse_conv.py:8-32).  Only the modules of the
sparse-convolution path exist; anything else raises ModuleNotFoundError as for any missing module.
"""
import importlib
import importlib.abc
import importlib.util
import sys

import warpconvnet_amd as _impl

_PREFIX = __name__ + "."
_TARGET = _impl.__name__


class _Alias(importlib.abc.MetaPathFinder, importlib.abc.Loader):
    def find_spec(self, fullname, path=None, target=None):
        if not fullname.startswith(_PREFIX):
            return None
        real = _TARGET + fullname[len(__name__):]
        try:
            if importlib.util.find_spec(real) is None:
                return None
        except ModuleNotFoundError:
            return None
        return importlib.util.spec_from_loader(fullname, self, is_package=True)

    def create_module(self, spec):
        real = importlib.import_module(_TARGET + spec.name[len(__name__):])
        # the import machinery is about to stamp the alias's spec onto the module it is handed;
        # the real module keeps its own (relative imports and reloads go by __spec__.parent)
        self._own_spec[id(real)] = real.__spec__
        return real

    def exec_module(self, module):  # the real module is already initialised
        own = self._own_spec.pop(id(module), None)
        if own is not None:
            module.__spec__ = own

    _own_spec = {}


sys.meta_path.insert(0, _Alias())
__path__ = []  # a package whose submodules all come from the finder above
__version__ = getattr(_impl, "__version__", "0")
