"""Loads the native pieces.  There is no fallback: if the HIP library or the
extension module has not been built, importing this module raises."""
import ctypes
import importlib
import os
import sys

import torch  # noqa: F401  (loads libc10 / libtorch / the HIP runtime first)

_PKG = os.path.dirname(os.path.abspath(__file__))
KERNEL_LIB = os.path.join(_PKG, "libtorchex_scatter.so")

if not os.path.exists(KERNEL_LIB):
    raise ImportError(
        f"{KERNEL_LIB} is missing: build it with `python torchex_amd/_build.py` "
        "(there is no CPU or PyTorch fallback for the scatter kernels)")

try:
    scatter_ext = importlib.import_module("torchex_amd.scatter_ext")
except ImportError as e:  # pragma: no cover
    raise ImportError(
        "torchex_amd.scatter_ext (the C++ extension module) failed to load: "
        f"{e}; build it with `python torchex_amd/_build.py`") from e

# The reference does `import scatter_ext` (torchex/operator_py/scatter_op.py:4);
# keep that spelling importable.
sys.modules.setdefault("scatter_ext", scatter_ext)
# The same for the modules its other wrappers import: `import ingroup_indices`
# (operator_py/ingroup_inds_op.py:4), `import dynamic_point_pool_ext`
# (operator_py/dynamic_point_pool_op.py:7), `import grid_hash_ext` (operator_py/grid_hash.py:2).
for _name in ("ingroup_indices", "dynamic_point_pool_ext", "grid_hash_ext"):
    sys.modules.setdefault(_name, getattr(scatter_ext, _name))


def cabi():
    """The C ABI as a ctypes handle (used by tests and tools, not by the ops)."""
    return ctypes.CDLL(KERNEL_LIB)
