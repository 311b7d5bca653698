"""``brt`` -- import-path alias of :mod:`brainstorm_amd`.

Code written against the reference (``import brt``, ``from brt.router import
ScatterRouter``, ``import brt._C.router as c_router``, ``from brt.jit import
make_jit_kernel`` ...) resolves to the modules of ``brainstorm_amd`` with the same
relative path; no module is loaded twice.
"""
import importlib
import importlib.abc
import importlib.util
import sys

import brainstorm_amd

_PREFIX, _TARGET = "brt", "brainstorm_amd"


class _AliasFinder(importlib.abc.MetaPathFinder, importlib.abc.Loader):
    def find_spec(self, fullname, path=None, target=None):
        if fullname == _PREFIX or not fullname.startswith(_PREFIX + "."):
            return None
        real = _TARGET + fullname[len(_PREFIX):]
        try:
            if importlib.util.find_spec(real) is None:
                return None
        except (ImportError, ValueError):
            return None
        return importlib.util.spec_from_loader(fullname, self)

    def create_module(self, spec):
        real = importlib.import_module(_TARGET + spec.name[len(_PREFIX):])
        return real  # the very same module object, registered under both names

    def exec_module(self, module):
        pass


sys.meta_path.insert(0, _AliasFinder())

# the package itself: same attributes, sub-packages resolved through the finder
from brainstorm_amd import *  # noqa: E402,F401,F403
from brainstorm_amd import Annotator, GridTensor, to_grid_tensor, to_torch_tensor  # noqa: E402,F401

__path__ = []  # sub-modules come from the finder, not from this directory
