"""Drop-in alias: `triton_kernels.<module>` resolves to `triton_amd.<module>`.

The reference library is imported as `triton_kernels` (`from triton_kernels.matmul import matmul`,
`from triton_kernels.topk import topk`, `from triton_kernels.numerics_details.mxfp import downcast_to_mxfp`, ...).
This package installs an import hook that maps every such module path onto the MI355X implementation in
`triton_amd`, so user code written against the reference runs unchanged.
"""
import importlib
import importlib.abc
import importlib.util
import sys

import triton_amd as _impl

__version__ = _impl.__version__


class _AliasFinder(importlib.abc.MetaPathFinder, importlib.abc.Loader):
    prefix = __name__ + "."

    def find_spec(self, fullname, path=None, target=None):
        if not fullname.startswith(self.prefix):
            return None
        real = "triton_amd." + fullname[len(self.prefix):]
        try:
            if importlib.util.find_spec(real) is None:
                return None
        except ModuleNotFoundError:
            return None
        return importlib.util.spec_from_loader(fullname, self)

    def create_module(self, spec):
        real = "triton_amd." + spec.name[len(self.prefix):]
        return importlib.import_module(real)

    def exec_module(self, module):
        pass


if not any(isinstance(f, _AliasFinder) for f in sys.meta_path):
    sys.meta_path.insert(0, _AliasFinder())
