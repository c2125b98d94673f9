"""MI355X-native voxel scatter-reductions with TorchEx's call surface.

``from torchex_amd import scatter_sum, scatter_mean, scatter_max, ScatterData,
TorchTimer`` -- the names the reference exports for this path
(``torchex/operator_py/__init__.py:2,6``).  Importing the package loads the HIP
kernel library and the ``scatter_ext`` extension module and raises if either is
missing.
"""
from .scatter_op import (ScatterData, getPreSum, ingroup_inds, scatter_max, scatter_mean, scatter_sum,
                         voxelize)
from .point_ops import GridHash, dynamic_point_pool, grid_hash_build, grid_hash_probe
from .timer import TorchTimer

__all__ = ['dynamic_point_pool', 'TorchTimer', 'ingroup_inds', 'scatter_sum', 'scatter_mean', 'scatter_max',
           'ScatterData', 'grid_hash_build', 'grid_hash_probe', 'GridHash']
