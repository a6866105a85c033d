"""flashbev_amd: fused camera->BEV pooling for AMD MI355X (gfx950).

Drop-in for the operator layer of yokosyun/FlashBEV's ``flashbevpool`` package
(flashbev/flashbevpool/__init__.py:3-6): same ``FlashBEVPool`` autograd function and
``flash_bevpool`` wrapper, backed by hand-written HIP kernels behind a C ABI
(``include/flashbev_hip.h``).  There is no CPU implementation in this package.
"""
from .flash_bevpool import FlashBEVPool, build_geometry_cache, flash_bevpool, release_workspaces, voxel_geometry
from .rig import create_projection_matrix
from .sampling_vt import SamplingVT
from .sampling_vt_ops import sampling_vt_pillarpool_fused

__all__ = ["FlashBEVPool", "flash_bevpool", "SamplingVT", "sampling_vt_pillarpool_fused", "create_projection_matrix",
           "voxel_geometry", "build_geometry_cache", "release_workspaces"]
__version__ = "0.1.0"
